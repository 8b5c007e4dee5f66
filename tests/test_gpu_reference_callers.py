"""Runs the reference's own test programs (tests/test_load_balance.cu:1-34,
test_sortedsearch.cu:1-33, test_reduce.cu:1-47, test_segreduce.cu:1-79,
test_join.cu:1-10, test_intervalexpand.cu:1-9, test_merge.cu:1-37), its
breadth-first-search demos and its tutorials,
compiled without any change against this library's headers: oracle/Makefile
builds them from where the reference tree lies into oracle/_ref/ (binaries
only; no source is copied).  Each program checks the device results against a
host loop of its own.  test_scan.cu and test_intervalmove.cu are not built:
they call the CUDA runtime by name.

The binaries exist only where they were built beside the reference tree; a
checkout without them skips these tests."""
import os
import pty
import re
import select
import subprocess
import time

import numpy as np
import pytest

pytestmark = pytest.mark.gpu
BIN = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))),
                   "oracle", "_ref")


# Programs named launcher_* are the same sources built with MGPU_HIP_LAUNCHER:
# the public templates then call the prebuilt kernels of libmgpu_hip.so where
# the arguments are ones its C layer covers.  With MGPU_HIP_LAUNCHER_REPORT in
# the environment such a program says on stderr when its first call goes
# there and, at exit, how many did.
_ENV = dict(os.environ, MGPU_HIP_LAUNCHER_REPORT="1")


def _run(name, limit=110):
    """Returns (exit status, stdout, stderr)."""
    path = os.path.join(BIN, name)
    if not os.path.exists(path):
        pytest.skip("oracle/_ref/%s was not built (no reference tree at build time)" % name)
    proc = subprocess.run([path], capture_output=True, text=True, timeout=limit, env=_ENV)
    return proc.returncode, proc.stdout, proc.stderr


def _launcher_calls(text):
    """The count a launcher_* program reports at exit (also when it is 0);
    None when there is no report (a program built without the dispatch layer,
    or one that was ended from outside)."""
    found = re.findall(r"mgpu launcher calls: (\d+)", text)
    return int(found[-1]) if found else None


def _run_for_a_while(name, seconds, enough=None):
    """Runs a program whose stdout is a terminal (so that it is flushed line by
    line) and returns (exit status or None, output).  The program is ended from
    outside -- SIGTERM, then SIGKILL if it does not go within 20 s -- once
    enough(output) is true or after `seconds`, whichever comes first: this is
    the one place where a test stops a process that may have kernels in
    flight (the two reference programs it is used for would otherwise run for
    hours).  The kernels in flight finish or are torn down with the process by
    the driver; nothing else shares the device with them."""
    path = os.path.join(BIN, name)
    if not os.path.exists(path):
        pytest.skip("oracle/_ref/%s was not built (no reference tree at build time)" % name)
    master, slave = pty.openpty()
    proc = subprocess.Popen([path], stdout=slave, stderr=slave, stdin=subprocess.DEVNULL,
                            env=_ENV)
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
        if enough is not None and enough(b"".join(chunks).decode(errors="replace")):
            break
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


@pytest.mark.parametrize("name", ["test_load_balance", "launcher_test_load_balance"])
def test_reference_test_load_balance(dev, name):
    # Prints one line per item of 200,030 and "ERROR AT" (then exit(0)) on a mismatch.
    # The launcher_ build defines MGPU_HIP_LAUNCHER: its load_balance_search
    # runs the prebuilt kernels of libmgpu_hip.so.
    code, out, err = _run(name)
    assert code == 0, err[-2000:]
    assert "ERROR" not in out
    lines = re.findall(r"^ *(\d+): +(\d+)$", out, flags=re.M)
    assert len(lines) == 200030
    assert lines[-1] == ("200029", str(200029 // 100))
    if name.startswith("launcher_"):
        assert _launcher_calls(err) == 1, err[-500:]


@pytest.mark.parametrize("name", ["test_sortedsearch", "launcher_test_sortedsearch"])
def test_reference_test_sortedsearch(dev, name):
    # Host asserts on every index (the build does not define NDEBUG).
    code, out, err = _run(name)
    assert code == 0, err[-2000:]
    if name.startswith("launcher_"):
        assert _launcher_calls(err) > 0, err[-500:]


@pytest.mark.parametrize("name", ["test_reduce", "launcher_test_reduce"])
def test_reference_test_reduce(dev, name):
    # 1,012 sizes from 1,000 to 23.4 M, reduce<192 x 11> and transform_reduce
    # against std::accumulate; exit(1) on a mismatch.  Both calls instantiate
    # in place whatever the build: one names a launch box, the other takes a
    # lambda.
    code, out, err = _run(name)
    assert code == 0, out[-2000:] + err[-2000:]
    assert "ERROR" not in out
    assert out.count("success") > 1000
    assert _launcher_calls(err) == (0 if name.startswith("launcher_") else None)


@pytest.mark.parametrize("name", ["test_segreduce", "launcher_test_segreduce"])
def test_reference_test_segreduce(dev, name):
    # 1,000 rounds of 10^8 items, each checked by a host loop: far more than a
    # test run has time for, so it is ended after a while and what it printed
    # until then is checked (it reports a mismatch and calls exit(0)).
    # The gate does not depend on how fast the host is: one complete round
    # without a mismatch passes; the run stops at three rounds or 60 s.
    code, out = _run_for_a_while(name, 60,
                                 enough=lambda text: text.count("passed") >= 3)
    print(out[-400:])
    assert code in (None, 0), out[-2000:]
    assert "error" not in out.lower()
    assert out.count("passed") >= 1, out[-2000:]
    # Its one call is transform_segreduce over a lambda, which instantiates in
    # place whatever the build (a call into the library would have announced
    # itself: the program is ended from outside, so no count is printed).
    assert "mgpu launcher: first call" not in out


@pytest.mark.parametrize("name", ["test_merge", "launcher_test_merge"])
def test_reference_test_merge(dev, name):
    # Sizes from 1,000 to 10^8 in steps of 10 %, each merged on the device and
    # with std::merge (the inputs are sorted on the host, which takes most of
    # the time at the large sizes); ended after a while like test_segreduce.
    # Stops at 60 sizes or 60 s; passes with no failure among at least the
    # first 25 sizes (1,000 to about 10,000 keys in all, a few milliseconds each on any
    # host: from one tile of the merge kernel to several).
    # merge is not among the calls the C layer covers: in place either way.
    code, out = _run_for_a_while(name, 60,
                                 enough=lambda text: text.count("SUCCESS") >= 60)
    print(out[-400:])
    assert code in (None, 0), out[-2000:]
    assert "FAILURE" not in out
    assert out.count("SUCCESS") >= 25, out[-2000:]


@pytest.mark.parametrize("prefix", ["", "launcher_"])
def test_reference_test_join_and_intervalexpand(dev, prefix):
    for name in ("test_join", "test_intervalexpand"):
        # test_join joins two empty inputs and test_intervalexpand only
        # creates a context: building and running them is the whole test.
        code, out, err = _run(prefix + name)
        assert code == 0, name + err[-2000:]


# ---- the breadth-first-search demos (demo/bfs.cu:1-92, bfs2.cu:1-113,
# bfs3.cu:1-134 with demo/graph.cxx:7-56) ------------------------------------
# They read a Matrix Market file at a fixed relative path (a graph that the
# reference does not ship), start at vertex 23, and write the level of every
# vertex to bfs.txt (bfs, bfs2) or print the size of every front (bfs3).  The
# tests give them a synthetic graph at that path in a scratch directory and
# compare with a breadth-first search in numpy.

def _synthetic_graph(tmp_path, num_vertices, num_edges, seed):
    rng = np.random.default_rng(seed)
    # A few hubs, many leaves, some vertices that nothing reaches.
    reach = int(num_vertices * 0.9)
    a = rng.integers(0, reach, num_edges)
    b = (rng.zipf(1.6, num_edges) + rng.integers(0, reach, num_edges)) % reach
    a[0], b[0] = 23, 24                         # the source has a neighbour
    folder = tmp_path / "demo" / "coPapersCiteseer"
    folder.mkdir(parents=True)
    with open(folder / "coPapersCiteseer.mtx", "w") as f:
        f.write("%%MatrixMarket matrix coordinate pattern symmetric\n")
        f.write("% synthetic\n")
        f.write("%d %d %d\n" % (num_vertices, num_vertices, num_edges))
        f.write("".join("%d %d\n" % (x + 1, y + 1) for x, y in zip(a, b)))
    # The loader stores every edge in both directions (graph.cxx:22-38).
    src = np.concatenate([a, b])
    dst = np.concatenate([b, a])
    order = np.lexsort((dst, src))
    src, dst = src[order], dst[order]
    starts = np.searchsorted(src, np.arange(num_vertices + 1))
    return starts, dst


def _bfs_levels(starts, dst, source):
    level = np.full(len(starts) - 1, -1, np.int64)
    level[source] = 0
    front = np.array([source])
    fronts = []
    while len(front):
        begin, end = starts[front], starts[front + 1]
        neighbours = np.concatenate([dst[b:e] for b, e in zip(begin, end)]) \
            if len(front) else np.zeros(0, np.int64)
        fresh = np.unique(neighbours[level[neighbours] == -1])
        level[fresh] = level[front[0]] + 1
        fronts.append((len(fresh), int((starts[fresh + 1] - starts[fresh]).sum())))
        front = fresh
    return level, fronts


def _run_demo(name, tmp_path):
    path = os.path.join(BIN, name)
    if not os.path.exists(path):
        pytest.skip("oracle/_ref/%s was not built (no reference tree at build time)" % name)
    proc = subprocess.run([path], capture_output=True, text=True, timeout=110,
                          cwd=str(tmp_path))
    assert proc.returncode == 0, proc.stdout[-2000:] + proc.stderr[-2000:]
    return proc.stdout


@pytest.mark.parametrize("name", ["bfs", "bfs2"])
def test_reference_demo_bfs_levels(dev, tmp_path, name):
    starts, dst = _synthetic_graph(tmp_path, 60_000, 400_000, 5)
    want, _ = _bfs_levels(starts, dst, 23)
    _run_demo(name, tmp_path)
    got = np.array([int(l.split(":")[1]) for l in open(tmp_path / "bfs.txt")])
    assert got.shape == want.shape
    assert (want == -1).any() and want.max() >= 3
    assert np.array_equal(got, want)


def test_reference_demo_bfs3_fronts(dev, tmp_path):
    starts, dst = _synthetic_graph(tmp_path, 60_000, 400_000, 6)
    _, fronts = _bfs_levels(starts, dst, 23)
    out = _run_demo("bfs3", tmp_path)
    got = [(int(v), int(e)) for v, e in re.findall(
        r"Front for level \d+ has (\d+) vertices and (\d+) edges", out)]
    assert got == fronts


# ---- the tutorials on the launch mechanism (tutorial/tut_01_transform.cu,
# tut_02_cta_launch.cu, tut_03_launch_box.cu, tut_04_launch_custom.cu) --------

def test_reference_tutorial_transform(dev):
    # Ten device threads print a line each.
    code, out, err = _run("tut_01_transform")
    assert code == 0, err[-2000:]
    threads = sorted(int(n) for n in re.findall(r"Thread (\d+) says the year is \d{4}", out))
    assert threads == list(range(10))


def test_reference_tutorial_cta_launch(dev):
    # A 16-thread CTA sums the first 16 squares through LDS.
    code, out, err = _run("tut_02_cta_launch")
    assert code == 0, err[-2000:]
    assert "Reduction of 16 elements is %d" % sum(i * i for i in range(1, 17)) in out


def test_reference_tutorial_launch_boxes(dev):
    # A box written for CUDA architectures resolves the way the reference
    # resolves it for its newest architecture (launch_box.hxx:31-45: sm_86 ->
    # 80 -> 75 -> 70 -> 62 -> 60 -> 53 -> 50 -> 35 -> 30 -> 21 -> 20, which
    # passes sm_52 by): tut_03's box to its sm_50 entry, tut_04's to sm_35.
    code, out, err = _run("tut_03_launch_box")
    assert code == 0, err[-2000:]
    assert "Standard launch box: nt = 256 vt = 8" in out
    code, out, err = _run("tut_04_launch_custom")
    assert code == 0, err[-2000:]
    assert "Custom launch box: nt = 128 mode = 2000 sizeof(type_t)=4" in out


def test_reference_tutorial_iterators(dev):
    # A computed sequence (Fibonacci numbers from a load iterator) is merged
    # with a strided one into a store iterator that also takes logarithms.
    import math
    code, out, err = _run("tut_05_iterators")
    assert code == 0, err[-2000:]
    fib = [0, 1]
    while len(fib) < 20:
        fib.append(fib[-1] + fib[-2])
    listed = {int(i): int(v) for i, v in re.findall(r"Fibonacci +(\d+) = +(\d+)", out)}
    assert listed == dict(enumerate(fib))
    merged = [(int(k), float(v)) for k, v in re.findall(r"log\( *(\d+)\) = ([-0-9.]+)", out)]
    assert [k for k, _ in merged] == sorted(fib + [50 + 500 * i for i in range(10)])
    for k, v in merged:
        assert abs(v - (math.log(k) if k else 0.0)) < 1e-5
