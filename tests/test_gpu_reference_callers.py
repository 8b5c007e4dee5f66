"""Runs the reference's own test programs (tests/test_load_balance.cu:1-34,
test_sortedsearch.cu:1-33, test_reduce.cu:1-47, test_segreduce.cu:1-79,
test_join.cu:1-10, test_intervalexpand.cu:1-9), compiled without any change
against this library's headers: tests/csrc/Makefile builds them from where the
reference tree lies into tests/csrc/reference_callers/ (binaries only; no
source is copied).  Each program checks the device results against a host loop
of its own.  test_scan.cu and test_intervalmove.cu are not built: they call
the CUDA runtime by name.

The binaries exist only where they were built beside the reference tree; a
checkout without them skips these tests."""
import os
import pty
import re
import select
import subprocess
import time

import pytest

pytestmark = pytest.mark.gpu
BIN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc",
                   "reference_callers")


def _run(name, limit=110):
    """Returns (exit status, stdout, stderr)."""
    path = os.path.join(BIN, name)
    if not os.path.exists(path):
        pytest.skip("reference_callers/%s was not built (no reference tree at build time)" % name)
    proc = subprocess.run([path], capture_output=True, text=True, timeout=limit)
    return proc.returncode, proc.stdout, proc.stderr


def _run_for_a_while(name, seconds):
    """Runs a program whose stdout is a terminal (so that it is flushed line by
    line), ends it after `seconds` and returns (exit status or None, output)."""
    path = os.path.join(BIN, name)
    if not os.path.exists(path):
        pytest.skip("reference_callers/%s was not built (no reference tree at build time)" % name)
    master, slave = pty.openpty()
    proc = subprocess.Popen([path], stdout=slave, stderr=slave, stdin=subprocess.DEVNULL)
    os.close(slave)
    chunks, deadline, code = [], time.time() + seconds, None
    while True:
        left = deadline - time.time()
        if left <= 0:
            break
        ready, _, _ = select.select([master], [], [], left)
        if not ready:
            break
        try:
            data = os.read(master, 65536)
        except OSError:             # the program closed its side: it has ended
            data = b""
        if not data:
            break
        chunks.append(data)
    if proc.poll() is None:
        proc.terminate()
        try:
            proc.wait(timeout=20)
        except subprocess.TimeoutExpired:
            proc.kill()
            proc.wait()
    else:
        code = proc.returncode
    os.close(master)
    return code, b"".join(chunks).decode(errors="replace")


def test_reference_test_load_balance(dev):
    # Prints one line per item of 200,030 and "ERROR AT" (then exit(0)) on a mismatch.
    code, out, err = _run("test_load_balance")
    assert code == 0, err[-2000:]
    assert "ERROR" not in out
    lines = re.findall(r"^ *(\d+): +(\d+)$", out, flags=re.M)
    assert len(lines) == 200030
    assert lines[-1] == ("200029", str(200029 // 100))


def test_reference_test_sortedsearch(dev):
    # Host asserts on every index (the build does not define NDEBUG).
    code, out, err = _run("test_sortedsearch")
    assert code == 0, err[-2000:]


def test_reference_test_reduce(dev):
    # 1,012 sizes from 1,000 to 23.4 M, reduce<192 x 11> and transform_reduce
    # against std::accumulate; exit(1) on a mismatch.
    code, out, err = _run("test_reduce")
    assert code == 0, out[-2000:] + err[-2000:]
    assert "ERROR" not in out
    assert out.count("success") > 1000


def test_reference_test_segreduce(dev):
    # 1,000 rounds of 10^8 items, each checked by a host loop: far more than a
    # test run has time for, so it is ended after a while and what it printed
    # until then is checked (it reports a mismatch and calls exit(0)).
    code, out = _run_for_a_while("test_segreduce", 25)
    assert code in (None, 0), out[-2000:]
    assert "error" not in out.lower()
    assert out.count("passed") >= 3, out[-2000:]


def test_reference_test_join_and_intervalexpand(dev):
    for name in ("test_join", "test_intervalexpand"):
        code, out, err = _run(name)
        assert code == 0, name + err[-2000:]
