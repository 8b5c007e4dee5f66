"""Pins the CPU oracle.  Every oracle function is checked against something
that does not share its formula: vectors recorded from the reference's own
host functions, the reference tests' expectations, closed forms, numpy/scipy
library routines and brute force on small inputs."""
import json
import math
import os

import numpy as np
import pytest

from moderngpu_amd import workloads

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


def _lengths(segments, count):
    return np.diff(np.append(np.asarray(segments, dtype=np.int64), count))


def _random_segments(rng, count, nseg, dup=0.3):
    s = np.zeros(nseg, dtype=np.int32)
    if nseg > 1:
        draws = rng.integers(0, count + 1, size=nseg - 1)
        if dup > 0 and nseg > 4:      # force runs of equal starts
            k = max(1, int(dup * (nseg - 1)))
            draws[rng.integers(0, nseg - 1, size=k)] = draws[rng.integers(0, nseg - 1, size=k)]
        s[1:] = np.sort(draws)
    return s


# --- merge path / partitions -------------------------------------------------

def test_merge_path_matches_reference_host_functions(oracle):
    g = json.load(open(os.path.join(GOLDEN, "reference_host_functions.json")))
    segs, count = g["segments"], g["count"]
    got = [oracle.merge_path(None, count, segs, d) for d in range(count + len(segs) + 1)]
    assert got == g["merge_path_upper_by_diag"]
    assert list(oracle.compute_merge_range(*g["compute_merge_range"]["args"])) == \
        g["compute_merge_range"]["result"]
    b = g["binary_search"]
    assert oracle.binary_search(b["keys"], b["key"], upper=False) == b["lower"]
    assert oracle.binary_search(b["keys"], b["key"], upper=True) == b["upper"]


def _explicit_merge_split(a, b, diag, upper):
    """Brute force: really merge, count how many of the first diag came from A."""
    i = j = 0
    for _ in range(diag):
        if j >= len(b):
            take_a = True
        elif i >= len(a):
            take_a = False
        else:
            take_a = (a[i] < b[j]) if upper else (a[i] <= b[j])
        if take_a:
            i += 1
        else:
            j += 1
    return i


@pytest.mark.parametrize("upper", [True, False])
def test_merge_path_brute_force(oracle, upper):
    rng = np.random.default_rng(1)
    for _ in range(60):
        na, nb = int(rng.integers(0, 40)), int(rng.integers(0, 40))
        a = np.sort(rng.integers(0, 25, size=na)).astype(np.int32)
        b = np.sort(rng.integers(0, 25, size=nb)).astype(np.int32)
        for diag in range(na + nb + 1):
            want = _explicit_merge_split(a, b, diag, upper)
            assert oracle.merge_path(a, na, b, diag, upper) == want


def test_lbs_partition_invariants(oracle):
    rng = np.random.default_rng(2)
    for _ in range(20):
        count = int(rng.integers(0, 5000))
        nseg = int(rng.integers(1, 600))
        segs = _random_segments(rng, count, nseg)
        spacing = int(rng.integers(1, 300))
        mp = oracle.lbs_partitions(count, segs, spacing)
        total = count + nseg
        assert mp.size == (total + spacing - 1) // spacing + 1
        assert mp[0] == 0 and mp[-1] == count
        assert np.all(np.diff(mp) >= 0)
        for i, a in enumerate(mp):
            diag = min(spacing * i, total)
            b = diag - a
            assert 0 <= b <= nseg
            if b > 0:
                assert segs[b - 1] <= a          # consumed starts are <= item
            if b < nseg and a > 0:
                assert a - 1 < segs[b]           # next start is after item a-1


def test_binary_search_matches_numpy(oracle):
    rng = np.random.default_rng(3)
    keys = np.sort(rng.integers(0, 100, size=500)).astype(np.int32)
    for key in range(-2, 103):
        assert oracle.binary_search(keys, key, upper=False) == np.searchsorted(keys, key, "left")
        assert oracle.binary_search(keys, key, upper=True) == np.searchsorted(keys, key, "right")
    got = oracle.binary_search_partitions(keys, 100, 7, upper=False)
    want = np.searchsorted(keys, np.minimum(np.arange(got.size) * 7, 100), "left")
    assert np.array_equal(got, want)


# --- load-balancing search ---------------------------------------------------

def test_lbs_reference_test_vector(oracle):
    # moderngpu tests/test_load_balance.cu:9-28: starts every 100, N = 200030.
    count, spacing = 200030, 100
    segs = np.arange(0, count, spacing, dtype=np.int32)
    assert segs.size == (count + spacing - 1) // spacing
    got = oracle.load_balance_search(count, segs)
    assert np.array_equal(got, np.arange(count) // spacing)


def test_lbs_closed_form_and_ranks(oracle):
    rng = np.random.default_rng(4)
    for _ in range(30):
        count = int(rng.integers(0, 3000))
        segs = _random_segments(rng, count, int(rng.integers(1, 400)))
        seg, rank = oracle.transform_lbs(count, segs)
        want = np.searchsorted(segs, np.arange(count), side="right") - 1
        assert np.array_equal(seg, want)
        assert np.array_equal(rank, np.arange(count) - segs[want])


def test_interval_expand_is_repeat(oracle):
    rng = np.random.default_rng(5)
    for dtype in (np.int32, np.int64, np.uint8, np.float64):
        count = 2500
        segs = _random_segments(rng, count, 300)
        vals = rng.integers(0, 200, size=300).astype(dtype)
        got = oracle.interval_expand(vals, count, segs)
        assert np.array_equal(got, np.repeat(vals, _lengths(segs, count)))


def test_interval_gather_scatter_move(oracle):
    rng = np.random.default_rng(6)
    count, nseg = 1200, 90
    segs = _random_segments(rng, count, nseg, dup=0.0)
    lens = _lengths(segs, count)
    # disjoint destination intervals: a shuffled packing of the segments.
    order = rng.permutation(nseg)
    dest = np.zeros(nseg, dtype=np.int64)
    dest[order] = np.concatenate([[0], np.cumsum(lens[order])[:-1]])
    dest = dest.astype(np.int32)
    src = rng.integers(0, 10 ** 6, size=count).astype(np.int32)
    seg = np.repeat(np.arange(nseg), lens)
    rank = np.arange(count) - segs[seg]
    assert np.array_equal(oracle.interval_gather(src, count, segs, dest), src[dest[seg] + rank])
    want = np.zeros(count, dtype=np.int32)
    want[dest[seg] + rank] = src
    assert np.array_equal(oracle.interval_scatter(src, count, segs, dest, count), want)
    gather = dest[::-1].copy()       # any valid source offsets of equal lengths
    lens_r = lens
    ok = gather.astype(np.int64) + lens_r <= count
    gather[~ok] = 0
    want = np.zeros(count, dtype=np.int32)
    want[dest[seg] + rank] = src[gather[seg] + rank]
    assert np.array_equal(oracle.interval_move(src, count, segs, dest, gather, count), want)


# --- segmented reduce --------------------------------------------------------

def test_segreduce_mod13_golden(oracle):
    g = json.load(open(os.path.join(GOLDEN, "segreduce_mod13.json")))
    for c in g["cases"]:
        segs = np.array(c["segments"], dtype=np.int32)
        want = np.array(c["expected"], dtype=np.int64)
        got = oracle.segreduce_mod13(c["count"], segs, init=g["init"])
        assert np.array_equal(got, want), c["seed"]
        vals = (np.arange(c["count"]) % 13).astype(np.int32)
        got2 = oracle.segreduce(vals, segs, "plus", g["init"])
        assert np.array_equal(got2, want), c["seed"]


def _numpy_segreduce(vals, segs, ufunc, init):
    count = vals.size
    lens = _lengths(segs, count)
    out = np.full(segs.size, init, dtype=vals.dtype)
    nz = lens > 0
    if nz.any():
        red = ufunc.reduceat(vals, segs[nz].astype(np.int64))
        out[nz] = red
    return out


@pytest.mark.parametrize("dtype", [np.int32, np.uint32, np.int64, np.uint64])
def test_segreduce_integers_vs_numpy(oracle, dtype):
    rng = np.random.default_rng(7)
    info = np.iinfo(dtype)
    for _ in range(10):
        count = int(rng.integers(1, 4000))
        segs = _random_segments(rng, count, int(rng.integers(1, 300)))
        vals = rng.integers(info.min, info.max, size=count, dtype=dtype, endpoint=True)
        with np.errstate(over="ignore"):
            assert np.array_equal(oracle.segreduce(vals, segs, "plus", 17),
                                  _numpy_segreduce(vals, segs, np.add, 17))
        assert np.array_equal(oracle.segreduce(vals, segs, "maximum", 3),
                              _numpy_segreduce(vals, segs, np.maximum, 3))
        assert np.array_equal(oracle.segreduce(vals, segs, "minimum", 5),
                              _numpy_segreduce(vals, segs, np.minimum, 5))


@pytest.mark.parametrize("dtype,tol", [(np.float32, 1e-5), (np.float64, 1e-12)])
def test_segreduce_float_vs_fsum(oracle, dtype, tol):
    rng = np.random.default_rng(8)
    count = 3000
    segs = _random_segments(rng, count, 120)
    vals = rng.random(count).astype(dtype)
    got = oracle.segreduce(vals, segs, "plus", -2.0)
    lens = _lengths(segs, count)
    for s in range(segs.size):
        if lens[s] == 0:
            assert got[s] == dtype(-2.0)
        else:
            exact = math.fsum(float(v) for v in vals[segs[s]:segs[s] + lens[s]])
            # serial summation bound: (terms) * eps * sum|x|, well inside tol
            # for these lengths (values are non-negative so sum|x| = exact).
            assert abs(got[s] - exact) <= lens[s] * np.finfo(dtype).eps * abs(exact)
            assert abs(got[s] - exact) <= tol * abs(exact) * max(1, lens[s] // 64 + 1)
    assert np.array_equal(oracle.segreduce(vals, segs, "maximum", -1.0),
                          _numpy_segreduce(vals, segs, np.maximum, dtype(-1.0)))
    assert np.array_equal(oracle.segreduce(vals, segs, "minimum", 9.0),
                          _numpy_segreduce(vals, segs, np.minimum, dtype(9.0)))


def test_segreduce_brute_force_and_init_rule(oracle):
    vals = np.array([5, 1, 4, 2, 8, 7], dtype=np.int32)
    segs = np.array([0, 0, 2, 2, 2, 5, 6, 6], dtype=np.int32)
    # segments: [], [5,1], [], [], [4,2,8], [7], [], []  -- init only in empties
    assert list(oracle.segreduce(vals, segs, "plus", -100)) == \
        [-100, 6, -100, -100, 14, 7, -100, -100]
    assert list(oracle.segreduce(vals, segs, "maximum", -100)) == \
        [-100, 5, -100, -100, 8, 7, -100, -100]
    assert list(oracle.segreduce(vals, segs, "minimum", 100)) == \
        [100, 1, 100, 100, 2, 7, 100, 100]


def test_max_min_tie_rule_signed_zero(oracle):
    # mgpu::max(a,b) = (a<b)?b:a keeps the left operand on ties.
    vals = np.array([0.0, -0.0, -0.0, 0.0], dtype=np.float32)
    segs = np.array([0, 2], dtype=np.int32)
    mx = oracle.segreduce(vals, segs, "maximum", 0.0)
    mn = oracle.segreduce(vals, segs, "minimum", 0.0)
    assert list(np.signbit(mx)) == [False, True]
    assert list(np.signbit(mn)) == [False, True]


# --- spmv ----------------------------------------------------------------------

def test_spmv_vs_scipy(oracle):
    import scipy.sparse as sp
    w = workloads.config4(seed=3, scale=4096)
    rows = w["segments"].size
    indptr = np.append(w["segments"].astype(np.int64), w["nnz"])
    lens = _lengths(w["segments"], w["nnz"])
    for dtype in (np.float32, np.float64):
        # The oracle adds serially in `dtype`: its distance from the exact
        # product is bounded by (terms + 1) * eps * sum|a x| (standard forward
        # bound for recursive summation, products rounded once).
        tol = (lens + 2) * np.finfo(dtype).eps
        m = w["matrix"].astype(dtype)
        x = w["vector"].astype(dtype)
        # scipy canonicalises index arrays in place: hand it copies.
        a = sp.csr_matrix((m.astype(np.float64), w["columns"].copy(), indptr.copy()),
                          shape=(rows, rows))
        want = a @ x.astype(np.float64)
        abs_a = sp.csr_matrix((np.abs(m.astype(np.float64)), w["columns"].copy(),
                               indptr.copy()), shape=(rows, rows))
        norm = abs_a @ np.abs(x.astype(np.float64))
        got = oracle.spmv(m, w["columns"], x, w["segments"])
        assert got.dtype == dtype
        assert np.all(np.abs(got - want) <= tol * norm + 1e-300)
        assert np.allclose(oracle.spmv_abs(m, w["columns"], x, w["segments"]), norm, rtol=1e-12)


def test_spmv_empty_rows_are_zero(oracle):
    m = np.array([2.0, 3.0], dtype=np.float32)
    c = np.array([1, 0], dtype=np.int32)
    x = np.array([10.0, 100.0], dtype=np.float32)
    segs = np.array([0, 0, 1, 2, 2], dtype=np.int32)
    assert list(oracle.spmv(m, c, x, segs)) == [0.0, 200.0, 30.0, 0.0, 0.0]


# --- scans ---------------------------------------------------------------------

def test_scan_vs_numpy(oracle):
    rng = np.random.default_rng(9)
    v = rng.integers(-50, 50, size=777).astype(np.int32)
    out, red = oracle.scan(v, "plus", 0, inclusive=True)
    assert np.array_equal(out, np.cumsum(v)) and red == v.sum()
    out, red = oracle.scan(v, "plus", 9, inclusive=False)
    assert out[0] == 9 and np.array_equal(out[1:], np.cumsum(v)[:-1])
    out, red = oracle.scan(v, "maximum", 0, inclusive=True)
    assert np.array_equal(out, np.maximum.accumulate(v))


def test_scan_reference_test_vector(oracle):
    """The reference's own scan test (tests/test_scan.cu:13-16): an exclusive
    plus-scan of 50,000 copies of 1.01 in double; element i is the i-fold
    running sum and the total is the 50,000-fold one.  Checked against the
    exact product with the rounding bound of i additions."""
    n = 50000
    v = np.full(n, 1.01, dtype=np.float64)
    out, red = oracle.scan(v, "plus", 0.0, inclusive=False)
    i = np.arange(n, dtype=np.float64)
    assert out[0] == 0.0
    assert np.all(np.abs(out - 1.01 * i) <= (i + 1) * np.finfo(np.float64).eps * 1.01 * (i + 1))
    assert abs(red - 1.01 * n) <= n * np.finfo(np.float64).eps * 1.01 * n
    # the running sum is strictly increasing and each step adds 1.01 to rounding
    assert np.all(np.abs(np.diff(out) - 1.01) <= 2 * np.spacing(out[1:]))


def test_scan_all_types_and_ops_vs_numpy(oracle):
    rng = np.random.default_rng(10)
    for dt in (np.int32, np.uint32, np.int64, np.uint64):
        v = rng.integers(0, 1 << 20, size=1234).astype(dt)
        out, red = oracle.scan(v, "plus", 0, inclusive=True)
        assert np.array_equal(out, np.cumsum(v, dtype=dt)) and red == v.sum(dtype=dt)
        out, red = oracle.scan(v, "plus", 0, inclusive=False)
        assert out[0] == 0 and np.array_equal(out[1:], np.cumsum(v, dtype=dt)[:-1])
        out, red = oracle.scan(v, "minimum", 0, inclusive=True)
        assert np.array_equal(out, np.minimum.accumulate(v)) and red == v.min()
        # exclusive max: the placed zero is not folded into later elements
        w = (v.astype(np.int64) - (1 << 21)).astype(np.int64) if dt == np.int64 else v
        out, red = oracle.scan(w, "maximum", 0, inclusive=False)
        assert out[0] == 0 and np.array_equal(out[1:], np.maximum.accumulate(w)[:-1])
        assert red == w.max()
    # wrap-around of integer sums
    v = np.full(5, np.iinfo(np.int32).max, dtype=np.int32)
    out, red = oracle.scan(v, "plus", 0, inclusive=True)
    assert np.array_equal(out, np.cumsum(v.astype(np.int64)).astype(np.int32))
    for dt in (np.float32, np.float64):
        v = rng.standard_normal(999).astype(dt)
        out, red = oracle.scan(v, "plus", 0, inclusive=True)
        exact = np.cumsum(v.astype(np.longdouble))
        bound = np.arange(1, v.size + 1) * np.finfo(dt).eps * np.cumsum(np.abs(v.astype(np.longdouble)))
        assert np.all(np.abs(out - exact) <= bound)
        out, red = oracle.scan(v, "maximum", 0, inclusive=True)
        assert np.array_equal(out, np.maximum.accumulate(v)) and red == v.max()


def test_reduce_reference_test_vector(oracle):
    """The reference's reduce test folds an array of ones with plus
    (tests/test_reduce.cu:14-20): the result is the count."""
    for n in (1000, 1010, 123457):
        out, red = oracle.scan(np.ones(n, dtype=np.int32), "plus", 0, inclusive=True)
        assert red == n
    out, red = oracle.scan(np.zeros(0, dtype=np.int32), "plus", 0, inclusive=False)
    assert red == 0 and out.size == 0


def test_lbs_segreduce_seg_plus_rank_closed_form(oracle):
    """f = seg + rank summed over a segment of length L is L * seg +
    L (L - 1) / 2 (mod 2^32); empty segments give init."""
    from moderngpu_amd import workloads
    for count, nseg, seed in ((100000, 1000, 0), (5000, 9000, 1), (1 << 20, 7, 2)):
        segs = workloads.reference_test_segments(count, nseg, seed)
        got = oracle.lbs_segreduce_seg_plus_rank(count, segs, init=-1)
        ends = np.append(segs[1:], count).astype(np.int64)
        L = ends - segs
        want = (L * np.arange(nseg, dtype=np.int64) + L * (L - 1) // 2)
        want = (want & 0xffffffff).astype(np.uint32).view(np.int32)
        want = np.where(L == 0, np.int32(-1), want)
        assert np.array_equal(got, want)


def test_cta_load_balance_structure(oracle):
    """The thread-by-thread tile search: per-item results agree with the
    device-wide search (pinned above), every item of the tile is produced by
    exactly one thread, a thread's merge bits count the items it takes, and
    consecutive threads' placements chain (thread t + 1 begins where the vt
    merge steps of thread t end)."""
    rng = np.random.default_rng(17)
    for nt, vt, count, nseg in ((64, 3, 1000, 300), (128, 7, 5000, 40), (64, 3, 700, 2000),
                                (128, 11, 20000, 3000)):
        segs = np.zeros(nseg, dtype=np.int32)
        segs[1:] = np.sort(rng.integers(0, count + 1, size=nseg - 1))
        want_seg, want_rank = oracle.transform_lbs(count, segs)
        nv = nt * vt
        tiles = (count + nseg + nv - 1) // nv
        seen = np.zeros(count, dtype=np.int32)
        for cta in range(tiles):
            r = oracle.cta_load_balance(count, segs, nt, vt, cta)
            idx, sg, rk = r["indices"], r["segments"], r["ranks"]
            valid = rk >= 0
            a_begin, a_end = int(r["range"][0]), int(r["range"][1])
            assert np.all((idx[valid] >= a_begin) & (idx[valid] < a_end))
            assert np.array_equal(sg[valid], want_seg[idx[valid]])
            assert np.array_equal(rk[valid], want_rank[idx[valid]])
            seen[idx[valid]] += 1
            flags = r["merge_flags"].astype(np.int64)
            taken = np.array([bin(int(f) & ((1 << vt) - 1)).count("1") for f in flags])
            # chaining: next thread's a_index = this thread's a_index + items taken
            assert np.array_equal(r["a_index"][1:], (r["a_index"] + taken)[:-1])
            # and its b_index advances by the starts passed (vt - items taken)
            assert np.array_equal(r["b_index"][1:], (r["b_index"] + vt - taken)[:-1])
            # the first thread starts at the tile's first item, in the open segment
            assert r["a_index"][0] == a_begin
            if a_begin < a_end:
                assert r["b_index"][0] + (1 if (flags[0] & 1) == 0 else 0) <= want_seg[a_begin]
        assert np.all(seen == 1)


def test_cta_load_balance_hand_example(oracle):
    """segments = {0, 3, 3, 7}, 10 items, tiles of 4 threads x 2: worked by
    hand from the merge order  s0 0 1 2 s1 s2 3 4 | 5 6 s3 7 8 9."""
    segs = np.array([0, 3, 3, 7], dtype=np.int32)
    # oracle_cta_load_balance needs nt, vt only as numbers: 4 x 2.
    r = oracle.cta_load_balance(10, segs, 4, 2, 0)
    # tile 0 = merged positions [0, 8): starts s0,s1,s2 and items 0..4
    assert list(r["range"][:2]) == [0, 5]
    assert list(r["a_index"]) == [0, 1, 3, 3]
    assert list(r["b_index"]) == [-1, 0, 0, 2]
    # thread 0: s0 (bit 0 clear), item 0 (bit 1 set), then peeks item 1 (bit 2 set)
    assert [int(f) & 3 for f in r["merge_flags"]] == [0b10, 0b11, 0b00, 0b11]
    r = oracle.cta_load_balance(10, segs, 4, 2, 1)
    assert list(r["range"][:2]) == [5, 10]
    assert list(r["a_index"]) == [5, 7, 8, 10]
    assert list(r["b_index"]) == [2, 2, 3, 3]


# --- work creation -------------------------------------------------------------

def _workcreate_numpy(created, segments):
    created = np.asarray(created, dtype=np.int64)
    who = np.flatnonzero(created > 0)
    counts = created[who]
    starts = np.cumsum(counts) - counts
    seg = np.searchsorted(np.asarray(segments), who, side="right") - 1
    rank = who - np.asarray(segments, dtype=np.int64)[seg] if who.size else who
    return int(counts.sum()), starts, who, seg, rank


def test_workcreate_vs_numpy(oracle):
    rng = np.random.default_rng(77)
    for count, nseg, keep in [(0, 0, 0.5), (0, 4, 0.5), (1, 1, 1.0), (50, 7, 0.5),
                              (5000, 300, 0.1), (5000, 4000, 0.9), (3000, 1, 0.0)]:
        segments = _random_segments(rng, count, nseg) if nseg else np.zeros(0, np.int32)
        created = rng.integers(1, 9, size=count).astype(np.int32)
        created[rng.random(count) >= keep] = 0
        created[rng.random(count) < 0.05] = -3        # creates nothing either
        got = oracle.workcreate(created, segments)
        want = _workcreate_numpy(created, segments)
        assert got[0] == want[0]
        for g, w in zip(got[1:], want[1:]):
            assert np.array_equal(g, w)


def test_workcreate_hand_example(oracle):
    # segments [0,3) [3,3) [3,7) [7,10); items 1, 3, 4 and 9 create 2, 1, 5, 4.
    created = [0, 2, 0, 1, 5, 0, 0, 0, 0, 4]
    got = oracle.workcreate(created, [0, 3, 3, 7])
    assert got[0] == 12
    assert got[1].tolist() == [0, 2, 3, 8]        # starts of the new segments
    assert got[2].tolist() == [1, 3, 4, 9]        # creating items
    assert got[3].tolist() == [0, 2, 2, 3]        # their segments
    assert got[4].tolist() == [1, 0, 1, 2]        # their ranks


def test_workcreate_bfs_vs_scipy(oracle):
    """The frontier loop of the reference's demo/bfs2.cu with the oracle as the
    engine: levels must be scipy's unweighted shortest path lengths."""
    import scipy.sparse as sp
    from scipy.sparse.csgraph import shortest_path
    rng = np.random.default_rng(5)
    n = 600
    rows = np.concatenate([np.arange(n - 60), rng.integers(0, n - 60, 500)])
    cols = np.concatenate([(np.arange(n - 60) + 1) % (n - 60), rng.integers(0, n - 60, 500)])
    a = sp.coo_matrix((np.ones(rows.size), (rows, cols)), shape=(n, n))
    a = ((a + a.T) > 0).astype(np.int8).tocsr()
    indptr, indices = a.indptr.astype(np.int32), a.indices.astype(np.int32)
    source = 23
    want = shortest_path(a, unweighted=True, indices=source)
    want = np.where(np.isinf(want), -1, want).astype(np.int32)

    level = np.full(n, -1, dtype=np.int32)
    level[source] = 0
    segments = np.zeros(1, dtype=np.int32)
    first_edge = np.array([indptr[source]], dtype=np.int32)
    count, depth = int(indptr[source + 1] - indptr[source]), 0
    while segments.size:
        seg, rank = oracle.transform_lbs(count, segments)
        created = np.zeros(count, dtype=np.int32)
        for i in range(count):                      # the upsweep functor
            w = indices[first_edge[seg[i]] + rank[i]]
            if level[w] == -1:
                level[w] = depth + 1
                created[i] = indptr[w + 1] - indptr[w]
        new_count, new_segments, src, src_seg, src_rank = oracle.workcreate(created, segments)
        w = indices[first_edge[src_seg] + src_rank]  # the downsweep functor
        assert np.array_equal(indptr[w + 1] - indptr[w], created[src])
        segments, first_edge, count = new_segments, indptr[w], new_count
        depth += 1
    assert np.array_equal(level, want)


# --- sorted search and join ------------------------------------------------------

def test_sorted_search_vs_numpy_and_reference_test_assertions(oracle):
    rng = np.random.default_rng(91)
    for n, h, hi in [(0, 10, 5), (10, 0, 5), (1000, 1000, 10000), (5000, 300, 50),
                     (300, 5000, 50), (2000, 2000, 3)]:
        needles = np.sort(rng.integers(0, hi + 1, size=n)).astype(np.int32)
        haystack = np.sort(rng.integers(0, hi + 1, size=h)).astype(np.int32)
        lower = oracle.sorted_search(needles, haystack, upper=False)
        upper = oracle.sorted_search(needles, haystack, upper=True)
        assert np.array_equal(lower, np.searchsorted(haystack, needles, side="left"))
        assert np.array_equal(upper, np.searchsorted(haystack, needles, side="right"))
        # what tests/test_sortedsearch.cu asserts for bounds_lower
        for i, index in enumerate(lower):
            assert index <= 0 or needles[i] > haystack[index - 1]
            assert index >= h or needles[i] <= haystack[index]


def test_inner_join_vs_brute_force(oracle):
    rng = np.random.default_rng(92)
    for na, nb, hi in [(0, 0, 3), (0, 7, 3), (7, 0, 3), (60, 80, 10), (200, 150, 1000),
                       (50, 50, 0)]:
        a = np.sort(rng.integers(0, hi + 1, size=na)).astype(np.int32)
        b = np.sort(rng.integers(0, hi + 1, size=nb)).astype(np.int32)
        want = [(i, j) for i in range(na) for j in range(nb) if a[i] == b[j]]
        got = oracle.inner_join(a, b)
        assert got.shape == (len(want), 2)
        assert [tuple(p) for p in got.tolist()] == want
