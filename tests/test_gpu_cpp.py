"""Runs the C++ callers written against the mgpu:: template API (same shape as
the reference's tests/test_segreduce.cu and tests/test_load_balance.cu, plus
user functors, user types, custom launch boxes and the work-creation engine).  They are compiled in-tree
by tests/csrc/Makefile and exit non-zero on any mismatch."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu
BIN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc")


def _run(name, *args):
    path = os.path.join(BIN, name)
    assert os.path.exists(path), "build tests/csrc first (make -C tests/csrc)"
    proc = subprocess.run([path] + [str(a) for a in args], capture_output=True,
                          text=True, timeout=110)
    assert proc.returncode == 0, proc.stdout[-2000:] + proc.stderr[-2000:]
    return proc.stdout


def test_reference_style_segreduce(dev):
    out = _run("test_segreduce", 10_000_000, 100_000, 5)
    assert "passed" in out
    out = _run("test_segreduce", 1_000_000, 100, 3)     # many short segments
    assert "passed" in out


def test_reference_style_load_balance(dev):
    assert "passed" in _run("test_load_balance")


def test_template_paths(dev):
    assert "all passed" in _run("test_templates")


def test_reference_style_scan_and_reduce(dev):
    assert "all passed" in _run("test_scan_reduce")


def test_reference_style_lbs_segreduce(dev):
    assert "all passed" in _run("test_lbs_segreduce", 4_000_000, 50_000)


def test_workcreate_engine_and_bfs(dev):
    assert "all passed" in _run("test_workcreate", 200_000)


def test_reference_style_sorted_search_and_join(dev):
    assert "all passed" in _run("test_join")


def test_api_surface_with_iterators_and_wide_types(dev):
    assert "all passed" in _run("test_api_surface")


def test_runtime_helpers(dev):
    assert "all passed" in _run("test_runtime")


def test_caller_built_segreduce_from_cta_blocks(dev):
    assert "all passed" in _run("test_cta_segreduce")


def test_templates_dispatch_to_the_prebuilt_library(dev):
    assert "all passed" in _run("test_launcher")


def test_nearest_cities_pipeline_on_the_reference_demo_data(dev):
    sample = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden",
                          "statecity_sample.csv")
    assert "all passed" in _run("test_cities", sample)
