"""Device-wide scan and reduce through the C ABI against the CPU checker.
Integers, max and min are bit-exact; floating-point sums are compared with
the reassociation bound (items * eps * sum of magnitudes), because tiles are
folded as (carry + (tile prefix)) rather than in one serial chain."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

SIZES = [0, 1, 63, 64, 65, 4095, 4096, 4097, 16384, 16385, 100000, (1 << 20) + 3,
         (1 << 24) + 4097]


def _dev(a, dev):
    a = np.ascontiguousarray(a)
    if a.dtype == np.uint32:
        return torch.from_numpy(a.view(np.int32)).to(dev)
    if a.dtype == np.uint64:
        return torch.from_numpy(a.view(np.int64)).to(dev)
    return torch.from_numpy(a).to(dev)


def _host(t, dtype):
    a = t.cpu().numpy()
    return a.view(dtype) if a.dtype != dtype else a


@pytest.mark.parametrize("dtype", [np.int32, np.uint32, np.int64, np.uint64])
@pytest.mark.parametrize("op", ["plus", "maximum", "minimum"])
def test_integer_scan_bit_exact(oracle, dev, dtype, op):
    import moderngpu_amd as m
    rng = np.random.default_rng(5)
    unsigned = dtype in (np.uint32, np.uint64)
    for n in SIZES:
        lo = 0 if unsigned else -(1 << 28)
        v = rng.integers(lo, 1 << 28, size=n).astype(dtype)
        for inclusive in (False, True):
            want, want_red = oracle.scan(v, op, 0, inclusive=inclusive)
            red = torch.full((1,), 77, dtype=_dev(v, dev).dtype, device=dev)
            got, _ = m.scan(_dev(v, dev), op, inclusive=inclusive, reduction=red,
                            unsigned=unsigned)
            torch.cuda.synchronize()
            assert np.array_equal(_host(got, dtype), want), (n, inclusive)
            assert _host(red, dtype)[0] == (want_red if n else 0), (n, inclusive)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_float_scan(oracle, dev, dtype):
    import moderngpu_amd as m
    rng = np.random.default_rng(6)
    eps = np.finfo(dtype).eps
    for n in SIZES:
        v = rng.standard_normal(n).astype(dtype)
        for inclusive in (False, True):
            got, _ = m.scan(_dev(v, dev), "plus", inclusive=inclusive)
            exact = np.cumsum(v.astype(np.longdouble))
            if not inclusive:
                exact = np.concatenate([[0], exact[:-1]])
            mag = np.cumsum(np.abs(v.astype(np.longdouble)))
            if not inclusive:
                mag = np.concatenate([[0], mag[:-1]])
            bound = (np.arange(n) + 2) * eps * mag
            assert np.all(np.abs(got.cpu().numpy() - exact) <= bound), (n, inclusive)
            # max/min: bit-exact
            want, want_red = oracle.scan(v, "maximum", 0, inclusive=inclusive)
            red = torch.zeros(1, dtype=got.dtype, device=dev)
            got, _ = m.scan(_dev(v, dev), "maximum", inclusive=inclusive, reduction=red)
            assert np.array_equal(got.cpu().numpy(), want), (n, inclusive)
            if n:
                assert red.item() == want_red


def test_scan_reference_test_vector(dev):
    """tests/test_scan.cu: exclusive plus-scan of 50,000 times 1.01 (double),
    reduction into host memory the device writes."""
    import moderngpu_amd as m
    n = 50000
    v = torch.full((n,), 1.01, dtype=torch.float64, device=dev)
    total = torch.zeros(1, dtype=torch.float64).pin_memory()
    out, _ = m.scan(v, "plus", inclusive=False, reduction=total)
    torch.cuda.synchronize()
    i = np.arange(n, dtype=np.float64)
    got = out.cpu().numpy()
    assert got[0] == 0.0
    assert np.all(np.abs(got - 1.01 * i) <= (i + 2) * np.finfo(np.float64).eps * 1.01 * (i + 1))
    assert abs(total.item() - 1.01 * n) <= n * np.finfo(np.float64).eps * 1.01 * n


def test_scan_in_place_and_lengths_to_starts(oracle, dev):
    """The use the path makes of scan: segment lengths -> segment starts,
    in place, total = item count."""
    import moderngpu_amd as m
    rng = np.random.default_rng(8)
    lengths = rng.geometric(1.0 / 64.0, size=300001).astype(np.int32)
    t = _dev(lengths, dev)
    red = torch.zeros(1, dtype=torch.int32, device=dev)
    m.scan(t, "plus", inclusive=False, out=t, reduction=red)
    want, total = oracle.scan(lengths, "plus", 0, inclusive=False)
    assert np.array_equal(t.cpu().numpy(), want) and red.item() == total == lengths.sum()


@pytest.mark.parametrize("dtype", [np.int32, np.int64, np.uint32, np.uint64])
def test_integer_reduce_bit_exact(oracle, dev, dtype):
    import moderngpu_amd as m
    rng = np.random.default_rng(7)
    unsigned = dtype in (np.uint32, np.uint64)
    for n in [1, 2, 64, 8191, 8192, 8193, 123457, (1 << 21) + 11]:
        v = rng.integers(0 if unsigned else -(1 << 28), 1 << 28, size=n).astype(dtype)
        for op in ("plus", "maximum", "minimum"):
            _, want = oracle.scan(v, op, 0, inclusive=True)
            got = m.reduce(_dev(v, dev), op, unsigned=unsigned)
            assert _host(got, dtype)[0] == want, (n, op)
    # reference test shape: all ones
    for n in (1000, 1010, 23456):
        got = m.reduce(torch.ones(n, dtype=torch.int32, device=dev), "plus")
        assert got.item() == n
    # empty input: nothing is written
    out = torch.full((1,), 5, dtype=torch.int32, device=dev)
    m.reduce(torch.zeros(0, dtype=torch.int32, device=dev), "plus", out=out)
    assert out.item() == 5


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_float_reduce(oracle, dev, dtype):
    import moderngpu_amd as m
    rng = np.random.default_rng(11)
    for n in [1, 100, 8193, 1 << 20]:
        v = rng.standard_normal(n).astype(dtype)
        got = m.reduce(_dev(v, dev), "plus").item()
        exact = float(np.sum(v.astype(np.longdouble)))
        assert abs(got - exact) <= (n + 2) * np.finfo(dtype).eps * float(np.abs(v).sum())
        assert m.reduce(_dev(v, dev), "maximum").item() == v.max()
        assert m.reduce(_dev(v, dev), "minimum").item() == v.min()


def test_scan_full_size_properties(dev):
    """2^26 int32 items: differences of the inclusive scan give the input
    back, and the last element equals the reduction."""
    import moderngpu_amd as m
    g = torch.Generator(device=dev); g.manual_seed(3)
    v = torch.randint(-1000, 1000, (1 << 26,), dtype=torch.int32, device=dev, generator=g)
    red = torch.zeros(1, dtype=torch.int32, device=dev)
    out, _ = m.scan(v, "plus", inclusive=True, reduction=red)
    assert torch.equal(out[1:] - out[:-1], v[1:]) and out[0] == v[0]
    assert out[-1] == red[0] == m.reduce(v, "plus")[0]
    assert red.item() == int(v.sum(dtype=torch.int64).item() & 0xffffffff) - (1 << 32) * (int(v.sum(dtype=torch.int64).item() & 0xffffffff) >> 31)
