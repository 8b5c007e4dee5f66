"""sorted_search and inner_join through the C ABI against the CPU checker
(integers: exact).  Shapes cover empty sides, long runs of equal keys that
span tiles, needles all in front of / behind the haystack, and the reference
test's own sizes (1000 needles and 1000 haystack keys in [0, 10000])."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _keys(rng, n, hi):
    return np.sort(rng.integers(0, hi + 1, size=n)).astype(np.int32)


@pytest.mark.parametrize("n,h,hi", [
    (0, 100, 10), (100, 0, 10), (1, 1, 0), (1000, 1000, 10000), (3072, 3072, 7),
    (100003, 7, 1 << 20), (7, 100003, 1 << 20), (200000, 300000, 50),
    (1 << 21, 1 << 20, 1 << 22), (1 << 20, 1 << 21, 1 << 12)])
def test_sorted_search_matches_oracle(oracle, dev, n, h, hi):
    import moderngpu_amd as m
    rng = np.random.default_rng(n * 31 + h)
    needles, haystack = _keys(rng, n, hi), _keys(rng, h, hi)
    for bounds in ("lower", "upper"):
        got = m.sorted_search(torch.from_numpy(needles).to(dev),
                              torch.from_numpy(haystack).to(dev), bounds)
        torch.cuda.synchronize()
        want = oracle.sorted_search(needles, haystack, upper=(bounds == "upper"))
        assert np.array_equal(got.cpu().numpy(), want), bounds


def test_sorted_search_disjoint_ranges(oracle, dev):
    import moderngpu_amd as m
    low = np.arange(0, 50000, dtype=np.int32)
    high = np.arange(100000, 180000, dtype=np.int32)
    for needles, haystack in ((low, high), (high, low)):
        for bounds in ("lower", "upper"):
            got = m.sorted_search(torch.from_numpy(needles).to(dev),
                                  torch.from_numpy(haystack).to(dev), bounds)
            want = oracle.sorted_search(needles, haystack, upper=(bounds == "upper"))
            assert np.array_equal(got.cpu().numpy(), want)


@pytest.mark.parametrize("na,nb,hi", [
    (0, 0, 3), (0, 50, 3), (50, 0, 3), (1000, 1000, 10000), (5000, 4000, 100),
    (300, 200, 0), (200000, 150000, 1 << 16), (1 << 20, 1 << 20, 1 << 20),
    # runs of equal b keys that go on far behind the tile in which they begin:
    # the match count of an a key is finished outside the tile's own keys
    (3000, 6000, 3), (20000, 20000, 50), (40, 100000, 1),
    # just past the size from which the search adds up the scan's partials:
    # no match at all, a handful of b keys, many a keys against one sample step
    (16385, 16385, 1 << 30), (16385, 3, 1), (70001, 9, 4),
    ((1 << 22) + 4097, 1000, 1 << 12)])
def test_inner_join_matches_oracle(oracle, dev, na, nb, hi):
    import moderngpu_amd as m
    rng = np.random.default_rng(na * 17 + nb)
    a, b = _keys(rng, na, hi), _keys(rng, nb, hi)
    got = m.inner_join(torch.from_numpy(a).to(dev), torch.from_numpy(b).to(dev))
    torch.cuda.synchronize()
    want = oracle.inner_join(a, b)
    assert tuple(got.shape) == want.shape
    assert np.array_equal(got.cpu().numpy(), want)


@pytest.mark.parametrize("n,h,hi", [
    (3 * (1 << 20) + 5, (1 << 21) + 3, 1 << 24),      # few ties
    ((1 << 22) + 1, 1023, 1 << 20),                   # a haystack shorter than one sample step
    (1025, (1 << 22) + 77, 1 << 20),                  # ... and needles
    ((1 << 21) + 1000, (1 << 21) + 24, 7),            # runs of equal keys far longer than a tile
    (5 << 20, 3 << 20, 1 << 30)])
def test_sorted_search_large_inputs_take_the_sampled_partition(dev, n, h, hi):
    """From 2^22 keys on the tile splits are searched over every 1,024th key
    first (and then inside one window of the inputs); results against numpy."""
    import moderngpu_amd as m
    rng = np.random.default_rng(n + 3 * h)
    needles, haystack = _keys(rng, n, hi), _keys(rng, h, hi)
    d_needles, d_haystack = torch.from_numpy(needles).to(dev), torch.from_numpy(haystack).to(dev)
    for bounds, side in (("lower", "left"), ("upper", "right")):
        got = m.sorted_search(d_needles, d_haystack, bounds)
        torch.cuda.synchronize()
        assert np.array_equal(got.cpu().numpy(), np.searchsorted(haystack, needles, side=side)), bounds


def test_sorted_search_large_disjoint_and_interleaved(dev):
    import moderngpu_amd as m
    n = (3 << 20) + 11
    low = np.arange(n, dtype=np.int32)
    high = np.arange(n, dtype=np.int32) + (1 << 28)
    even, odd = 2 * np.arange(n, dtype=np.int32), 2 * np.arange(n, dtype=np.int32) + 1
    for needles, haystack in ((low, high), (high, low), (even, odd), (odd, even), (even, even)):
        for bounds, side in (("lower", "left"), ("upper", "right")):
            got = m.sorted_search(torch.from_numpy(needles).to(dev),
                                  torch.from_numpy(haystack).to(dev), bounds)
            assert np.array_equal(got.cpu().numpy(),
                                  np.searchsorted(haystack, needles, side=side))


def test_inner_join_large(oracle, dev):
    import moderngpu_amd as m
    rng = np.random.default_rng(77)
    a, b = _keys(rng, (1 << 22) + 9, 1 << 22), _keys(rng, (1 << 21) + 1, 1 << 22)
    got = m.inner_join(torch.from_numpy(a).to(dev), torch.from_numpy(b).to(dev))
    want = oracle.inner_join(a, b)
    assert tuple(got.shape) == want.shape
    assert np.array_equal(got.cpu().numpy(), want)
