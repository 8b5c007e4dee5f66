"""Runs the C++ callers written against the mgpu:: template API (same shape as
the reference's tests/test_segreduce.cu and tests/test_load_balance.cu, plus
user functors, user types, custom launch boxes and the work-creation engine).  They are compiled in-tree
by tests/csrc/Makefile and exit non-zero on any mismatch."""
import os
import re
import subprocess

import pytest

pytestmark = pytest.mark.gpu
BIN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc")


def _run(name, *args, report=False):
    path = os.path.join(BIN, name)
    assert os.path.exists(path), "build tests/csrc first (make -C tests/csrc)"
    env = dict(os.environ, MGPU_HIP_LAUNCHER_REPORT="1") if report else None
    proc = subprocess.run([path] + [str(a) for a in args], capture_output=True,
                          text=True, timeout=110, env=env)
    assert proc.returncode == 0, proc.stdout[-2000:] + proc.stderr[-2000:]
    return (proc.stdout, proc.stderr) if report else proc.stdout


def _launcher_calls(stderr):
    """The count a program built with MGPU_HIP_LAUNCHER reports at exit (also
    when it is 0); None when there is no report, i.e. the program was built
    without the dispatch layer."""
    found = re.findall(r"mgpu launcher calls: (\d+)", stderr)
    return int(found[-1]) if found else None


# The same callers built with MGPU_HIP_LAUNCHER: the public templates call the
# prebuilt kernels of libmgpu_hip.so wherever the arguments are ones its C
# layer covers, and instantiate in place elsewhere.  Each program has to pass
# as before and report how many of its calls went to the library.
@pytest.mark.parametrize("name,args,expected", [
    # transform_segreduce over a lambda: nothing the C layer could take
    ("test_segreduce", (10_000_000, 100_000, 3), "none"),
    ("test_load_balance", (), "some"),
    # every call names a launch box or uses a value type of its own
    ("test_scan_reduce", (), "none"),
    ("test_join", (), "some"),
    ("test_lbs_segreduce", (4_000_000, 50_000), "any"),
])
def test_callers_through_the_dispatch_layer(dev, name, args, expected):
    out, err = _run("launcher_" + name, *args, report=True)
    assert "passed" in out
    calls = _launcher_calls(err)
    assert calls is not None, "no report: not built with MGPU_HIP_LAUNCHER? " + err[-500:]
    print(name, "calls into libmgpu_hip.so:", calls)
    if expected == "some":
        assert calls > 0, err[-500:]
    if expected == "none":
        assert calls == 0, err[-500:]


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
