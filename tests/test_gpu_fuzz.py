"""Many small random shapes through the C ABI against the CPU checker: sizes
around one to a few tiles, segment starts with heavy duplication (runs of
empty segments), starts equal to count, single segments, no items.  Integer
types only, so everything must match bit for bit.  The seeds are fixed: a
failure names its case."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

SIZES = [0, 1, 2, 63, 64, 65, 255, 256, 257, 2047, 2048, 2049, 4095, 4096, 4097,
         6079, 6080, 6081, 6143, 6144, 6145, 8127, 8128, 8129, 8191, 8192, 12287, 12288,
         16255, 16256, 16257, 20000, 50001]


def _case(rng):
    count = int(rng.choice(SIZES)) + int(rng.integers(0, 3))
    kind = int(rng.integers(0, 6))
    if kind == 0:
        nseg = 1
    elif kind == 1:
        nseg = int(rng.integers(1, 8))
    elif kind == 2:
        nseg = max(1, count // int(rng.integers(1, 40)))
    elif kind == 3:
        nseg = count + int(rng.integers(1, 300))          # more segments than items
    elif kind == 4:
        nseg = int(rng.integers(1, 5000))
    else:
        nseg = int(rng.choice(SIZES)) + 1
    starts = np.zeros(nseg, dtype=np.int32)
    if nseg > 1:
        draws = rng.integers(0, count + 1, size=nseg - 1)
        mode = int(rng.integers(0, 4))
        if mode == 1:                                     # few distinct starts
            draws = rng.choice(rng.integers(0, count + 1, size=4), size=nseg - 1)
        elif mode == 2:                                   # everything at the end
            draws[:] = count
        elif mode == 3:                                   # on multiples of 64
            draws = (draws // 64) * 64
        starts[1:] = np.sort(draws)
    return count, starts


@pytest.mark.parametrize("seed", range(40))
def test_segreduce_lbs_scan_fuzz(oracle, dev, seed):
    import moderngpu_amd as m
    rng = np.random.default_rng(1000 + seed)
    for _ in range(6):
        count, starts = _case(rng)
        tag = (seed, count, starts.size)
        segs = torch.from_numpy(starts).to(dev)
        dtype = [np.int32, np.int64][int(rng.integers(0, 2))]
        op = ["plus", "maximum", "minimum"][int(rng.integers(0, 3))]
        values = rng.integers(-1000, 1000, size=count).astype(dtype)
        got = m.segreduce(torch.from_numpy(values).to(dev), segs, op, -77)
        assert np.array_equal(got.cpu().numpy(),
                              oracle.segreduce(values, starts, op, -77)), ("segreduce",) + tag
        got = m.load_balance_search(count, segs)
        want = oracle.load_balance_search(count, starts)
        assert np.array_equal(got.cpu().numpy(), want), ("lbs",) + tag
        seg, rank = m.transform_lbs(count, segs)
        assert np.array_equal(seg.cpu().numpy(), want), ("transform_lbs seg",) + tag
        assert np.array_equal(rank.cpu().numpy(),
                              np.arange(count, dtype=np.int64) - starts[want].astype(np.int64)
                              if count else np.zeros(0)), ("transform_lbs rank",) + tag
        per_seg = rng.integers(0, 1 << 20, size=starts.size).astype(np.int32)
        got = m.interval_expand(torch.from_numpy(per_seg).to(dev), count, segs)
        assert np.array_equal(got.cpu().numpy(),
                              oracle.interval_expand(per_seg, count, starts)), ("expand",) + tag
        got, _ = m.scan(torch.from_numpy(values).to(dev), op, inclusive=bool(seed & 1))
        assert np.array_equal(got.cpu().numpy(),
                              oracle.scan(values, op, 0, inclusive=bool(seed & 1))[0]), \
            ("scan",) + tag
        created = rng.integers(-1, 4, size=count).astype(np.int32)
        got = m.workcreate(torch.from_numpy(created).to(dev), segs)
        want = oracle.workcreate(created, starts)
        assert got[0] == want[0], ("workcreate count",) + tag
        for g, x in zip(got[1:], want[1:]):
            assert np.array_equal(g.cpu().numpy(), x), ("workcreate",) + tag


@pytest.mark.parametrize("seed", range(16))
def test_join_fuzz_many_keys(oracle, dev, seed):
    """inner_join past the size from which the search kernel adds up the
    partials of the scan behind it, with runs of equal keys from none to far
    longer than the window in which the upper bound is looked for first."""
    import moderngpu_amd as m
    rng = np.random.default_rng(777000 + seed)
    for _ in range(4):
        n = int(rng.choice([16384, 16385, 20000, 50000, 131072, 300001])) + int(rng.integers(0, 5000))
        h = int(rng.choice([1, 7, 3000, 16385, 50000, 131072, 300001])) + int(rng.integers(0, 5000))
        run = float(rng.choice([0.01, 0.5, 1, 3, 6, 7, 8, 12, 40, 500]))
        hi = max(0, int(h / run))
        if n * run > 3e6:
            n = int(3e6 / run)
        a = np.sort(rng.integers(0, hi + 1, size=n)).astype(np.int32)
        b = np.sort(rng.integers(0, hi + 1, size=h)).astype(np.int32)
        got = m.inner_join(torch.from_numpy(a).to(dev), torch.from_numpy(b).to(dev))
        want = oracle.inner_join(a, b)
        assert tuple(got.shape) == want.shape, (seed, n, h, hi)
        assert np.array_equal(got.cpu().numpy(), want), (seed, n, h, hi)


@pytest.mark.parametrize("seed", range(20))
def test_search_and_join_fuzz(oracle, dev, seed):
    import moderngpu_amd as m
    rng = np.random.default_rng(2000 + seed)
    for _ in range(6):
        n = int(rng.choice(SIZES[:22])) + int(rng.integers(0, 3))
        h = int(rng.choice(SIZES[:22])) + int(rng.integers(0, 3))
        hi = int(rng.choice([0, 1, 5, 100, 10000, 1 << 30]))
        a = np.sort(rng.integers(0, hi + 1, size=n)).astype(np.int32)
        b = np.sort(rng.integers(0, hi + 1, size=h)).astype(np.int32)
        da, db = torch.from_numpy(a).to(dev), torch.from_numpy(b).to(dev)
        for bounds in ("lower", "upper"):
            got = m.sorted_search(da, db, bounds)
            assert np.array_equal(got.cpu().numpy(),
                                  oracle.sorted_search(a, b, upper=(bounds == "upper"))), \
                (seed, n, h, hi, bounds)
        if n * h < 4_000_000 or hi > 100:
            got = m.inner_join(da, db)
            assert np.array_equal(got.cpu().numpy(), oracle.inner_join(a, b)), (seed, n, h, hi)


def test_large_random_shapes(oracle, dev):
    """Hundreds of tiles per call: counts up to 2 * 10^6 with few, many, far too
    many and Zipf-distributed segments, for the search (both outputs), interval
    expand on 4- and 8-byte values and an int32 segmented sum."""
    import moderngpu_amd as m
    rng = np.random.default_rng(77)
    for case in range(60):
        count = int(rng.integers(0, 2_000_000))
        kind = case % 5
        if kind == 0:
            nseg = int(rng.integers(1, 50))
        elif kind == 1:
            nseg = max(1, count // int(rng.integers(1, 64)))
        elif kind == 2:
            nseg = int(rng.integers(1, 3_000_000))
        elif kind == 3:
            nseg = max(1, count // 3)
        else:
            nseg = int(rng.integers(1, 20000))
        starts = np.zeros(nseg, dtype=np.int32)
        if nseg > 1:
            if case % 7 == 0:
                lens = np.minimum(rng.zipf(1.3, size=nseg), 1 << 16).astype(np.int64)
                lens = (lens * (count / max(1, lens.sum()))).astype(np.int64)
                starts[1:] = np.minimum(np.cumsum(lens)[:-1], count)
            else:
                starts[1:] = np.sort(rng.integers(0, count + 1, size=nseg - 1))
        tag = (case, count, nseg)
        segs = torch.from_numpy(starts).to(dev)
        want = oracle.load_balance_search(count, starts)
        got = m.load_balance_search(count, segs).cpu().numpy()
        assert np.array_equal(got, want), ("lbs",) + tag
        seg, rank = m.transform_lbs(count, segs)
        assert np.array_equal(seg.cpu().numpy(), want), ("transform_lbs seg",) + tag
        assert np.array_equal(rank.cpu().numpy(),
                              np.arange(count, dtype=np.int64) - starts[want]), \
            ("transform_lbs rank",) + tag
        for dtype, top in ((np.int32, 1 << 30), (np.int64, 1 << 60)):
            per_seg = rng.integers(0, top, size=nseg).astype(dtype)
            got = m.interval_expand(torch.from_numpy(per_seg).to(dev), count, segs)
            assert np.array_equal(got.cpu().numpy(),
                                  oracle.interval_expand(per_seg, count, starts)), \
                ("expand", dtype.__name__) + tag
        vals = rng.integers(-1000, 1000, size=count).astype(np.int32)
        got = m.segreduce(torch.from_numpy(vals).to(dev), segs, "plus", -5)
        assert np.array_equal(got.cpu().numpy(),
                              oracle.segreduce(vals, starts, "plus", -5)), ("segreduce",) + tag


@pytest.mark.parametrize("seed", range(24))
def test_short_segments_fuzz(oracle, dev, seed):
    """Inputs whose tiles hold more segment starts than threads: segments of a
    few items, of lengths around the 32 items up to which a thread folds a
    segment by itself, and short ones with a long one here and there (those
    tiles fall back to the scan).  A few tiles each, with and without the
    partition kernel; integer types, bit for bit."""
    import moderngpu_amd as m
    rng = np.random.default_rng(7000 + seed)
    for _ in range(5):
        nseg = int(rng.integers(300, 30_000))
        kind = int(rng.integers(0, 4))
        if kind == 0:
            lens = np.full(nseg, int(rng.integers(1, 13)))
        elif kind == 1:
            lens = rng.integers(0, int(rng.choice([2, 4, 31, 32, 33, 34, 48])) + 1, size=nseg)
        elif kind == 2:
            lens = (rng.random(nseg) < 0.6).astype(np.int64)
            where = rng.integers(0, nseg, size=int(rng.integers(1, 6)))
            lens[where] = rng.integers(33, 9000, size=where.size)
        else:
            lens = rng.integers(0, 3, size=nseg)
            lens[rng.integers(0, nseg, size=nseg // 50 + 1)] = 32
            lens[rng.integers(0, nseg, size=3)] = 33
        starts = np.concatenate([[0], np.cumsum(lens)[:-1]]).astype(np.int32)
        count = int(lens.sum()) + int(rng.integers(0, 2)) * int(rng.integers(0, 100))
        tag = (seed, kind, count, nseg)
        segs = torch.from_numpy(starts).to(dev)
        dtype = [np.int32, np.int64, np.uint32][int(rng.integers(0, 3))]
        op = ["plus", "maximum", "minimum"][int(rng.integers(0, 3))]
        values = rng.integers(0, 2000, size=count).astype(dtype)
        want = oracle.segreduce(values, starts, op, 5)
        dev_values = torch.from_numpy(values.view(np.int32) if dtype == np.uint32
                                      else values).to(dev)
        for phases in (7, 7 | 8):
            got = m.segreduce(dev_values, segs, op, 5, unsigned=dtype == np.uint32,
                              phases=phases).cpu().numpy()
            got = got.view(np.uint32) if dtype == np.uint32 else got
            assert np.array_equal(got, want), ("segreduce", phases, np.dtype(dtype).name, op) + tag
        got = m.lbs_segreduce_seg_plus_rank(count, segs, init=-1)
        assert np.array_equal(got.cpu().numpy(),
                              oracle.lbs_segreduce_seg_plus_rank(count, starts, init=-1)), \
            ("lbs_segreduce",) + tag
