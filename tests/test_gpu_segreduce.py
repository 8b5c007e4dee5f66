"""Segmented reduction through the C ABI against the CPU oracle: bit-exact for
integer types and for max/min of floats; for floating sums within the stated
tolerance of an exact (math.fsum / float64) sum and of the oracle's serial sum.

Tolerances (relative to sum |x| of the segment; reassociation only):
    float32 sums 1e-5, float64 sums 1e-12.
"""
import json
import os

import numpy as np
import pytest

from util import lengths_of, random_segments, segment_layouts

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(__file__), "golden")
TOL = {np.dtype(np.float32): 1e-5, np.dtype(np.float64): 1e-12}


def _dev(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _gpu_segreduce(values, segs, op, init, phases=7):
    import torch
    import moderngpu_amd as m
    unsigned = values.dtype in (np.uint32, np.uint64)
    v = values.view(np.int32 if values.dtype == np.uint32 else np.int64) if unsigned else values
    # Poison the output so segments nobody writes are noticed.
    out = torch.full((segs.size,), 0x5a5a5a5a if v.dtype.kind in "iu" else float("nan"),
                     dtype=_dev(v[:0]).dtype, device="cuda")
    m.segreduce(_dev(v), _dev(segs), op, init, out=out, unsigned=unsigned, phases=phases)
    got = out.cpu().numpy()
    return got.view(values.dtype) if unsigned else got


def _abs_sums(values, segs):
    lens = lengths_of(segs, values.size)
    out = np.zeros(segs.size)
    nz = lens > 0
    if nz.any() and values.size:
        out[nz] = np.add.reduceat(np.abs(values.astype(np.float64)), segs[nz].astype(np.int64))
    return out


def _check(values, segs, op, init, oracle, name="", phases=7):
    got = _gpu_segreduce(values, segs, op, init, phases)
    want = oracle.segreduce(values, segs, op, init)
    if values.dtype.kind == "f" and op == "plus":
        # "exact": extended-precision (x87 long double) sum of the same inputs.
        lens = lengths_of(segs, values.size)
        exact = np.zeros(segs.size, dtype=np.longdouble)
        if values.size and (lens > 0).any():
            exact[lens > 0] = np.add.reduceat(values.astype(np.longdouble),
                                              segs[lens > 0].astype(np.int64))
        bound = TOL[values.dtype] * _abs_sums(values, segs)
        assert np.array_equal(got[lens == 0], want[lens == 0]), name
        assert np.all(np.abs(got.astype(np.longdouble) - exact)[lens > 0] <= (bound + 1e-300)[lens > 0]), name
        # and next to the oracle's serial sum in the same type
        assert np.all(np.abs(got.astype(np.float64) - want.astype(np.float64)) <= 4 * bound + 1e-300), name
    else:
        assert got.tobytes() == want.tobytes(), (name, op, values.dtype)


def test_golden_mod13(dev, oracle):
    """The reference test's shape: transform_segreduce of index % 13, int32 +,
    init -1, starts from std::mt19937 (tests/test_segreduce.cu:16-49)."""
    import moderngpu_amd as m
    g = json.load(open(os.path.join(GOLDEN, "segreduce_mod13.json")))
    for c in g["cases"]:
        segs = np.array(c["segments"], dtype=np.int32)
        want = np.array(c["expected"], dtype=np.int32)
        got = m.transform_segreduce_mod13(c["count"], _dev(segs), g["init"]).cpu().numpy()
        assert np.array_equal(got, want), c["seed"]
        vals = (np.arange(c["count"]) % 13).astype(np.int32)
        assert np.array_equal(_gpu_segreduce(vals, segs, "plus", g["init"]), want)


def test_mod13_large_closed_form(dev):
    """The reference test's own size class: 10^7 items in 100 segments, so
    every segment spans many tiles (exercises the carry spine)."""
    import moderngpu_amd as m
    from moderngpu_amd import workloads
    count = 10_000_000
    for seed in range(3):
        segs = workloads.reference_test_segments(count, 100, seed)
        got = m.transform_segreduce_mod13(count, _dev(segs), -1).cpu().numpy()

        def prefix(n):
            n = n.astype(np.int64)
            r = n % 13
            return 78 * (n // 13) + r * (r - 1) // 2
        ends = np.append(segs[1:], count)
        want = np.where(ends > segs, prefix(ends) - prefix(segs), -1).astype(np.int32)
        assert np.array_equal(got, want)


@pytest.mark.parametrize("dtype", [np.int32, np.uint32, np.int64, np.uint64,
                                   np.float32, np.float64])
@pytest.mark.parametrize("op", ["plus", "maximum", "minimum"])
def test_layouts_all_types(dev, oracle, dtype, op):
    import moderngpu_amd as m
    rng = np.random.default_rng(21)
    code = {np.int32: 0, np.uint32: 1, np.int64: 2, np.uint64: 3,
            np.float32: 4, np.float64: 5}[dtype]
    nv = m.segreduce_tile_size(code)
    for name, count, segs in segment_layouts(rng, nv):
        if np.dtype(dtype).kind == "f":
            values = (rng.standard_normal(count) * 100).astype(dtype)
            init = dtype(-7.5)
        else:
            info = np.iinfo(dtype)
            values = rng.integers(info.min, info.max, size=count, dtype=dtype, endpoint=True)
            init = 42
        # as the call runs (small calls: tiles that find their own splits),
        # and with the partition kernel in front whatever the size
        _check(values, segs, op, init, oracle, name)
        _check(values, segs, op, init, oracle, name + "/partitioned", phases=7 | 8)


@pytest.mark.parametrize("dtype", [np.int32, np.uint32, np.int64, np.uint64,
                                   np.float32, np.float64])
def test_short_segments_2p22(dev, oracle, dtype):
    """2^22 items in segments of 1, 3 and 8 items (tiles with more starts than
    threads, a thousand or more of them) and of 0 to 40 items at random, for
    every value type: plus and maximum against the CPU loop."""
    rng = np.random.default_rng(24)
    count = 1 << 22
    if np.dtype(dtype).kind == "f":
        values = (rng.standard_normal(count) * 100).astype(dtype)
    else:
        info = np.iinfo(dtype)
        values = rng.integers(info.min, info.max, size=count, dtype=dtype, endpoint=True)
    layouts = [("len%d" % k, np.arange(0, count, k, dtype=np.int32)) for k in (1, 3, 8)]
    lens = rng.integers(0, 41, size=count // 16)
    starts = np.concatenate([[0], np.cumsum(lens)[:-1]])
    layouts.append(("mixed", starts[starts <= count].astype(np.int32)))
    for name, segs in layouts:
        _check(values, segs, "plus", 3, oracle, name)
        _check(values, segs, "maximum", 3, oracle, name)


def test_float_specials(dev, oracle):
    # +0/-0 ties and infinities through max/min must match the host loop's
    # left-operand-wins rule bit for bit.
    rng = np.random.default_rng(22)
    count = 20000
    segs = random_segments(rng, count, 700)
    for dtype in (np.float32, np.float64):
        pool = np.array([0.0, -0.0, 1.0, -1.0, np.inf, -np.inf, 3.5], dtype=dtype)
        values = pool[rng.integers(0, pool.size, size=count)]
        for op in ("maximum", "minimum"):
            _check(values, segs, op, dtype(2.0), oracle, "specials")


def test_config1(dev, oracle):
    from moderngpu_amd import workloads
    w = workloads.config1()
    _check(w["values"], w["segments"], "plus", 0, oracle, "config1")
    # the reference test's closed upper bound: a start may equal count
    segs = workloads.reference_test_segments(w["values"].size, 10000, 42)
    _check(w["values"], segs, "plus", -1, oracle, "config1_closed")


def test_config2_scaled(dev, oracle):
    from moderngpu_amd import workloads
    w = workloads.config2(scale=8)
    _check(w["values"], w["segments"], "plus", 0.0, oracle, "config2/8")


@pytest.mark.parametrize("kind", ["f64max", "i64sum"])
def test_config5_scaled(dev, oracle, kind):
    from moderngpu_amd import workloads
    w = workloads.config5(scale=8, kind=kind)
    _check(w["values"], w["segments"], w["op"], w["init"], oracle, "config5/8")


def test_spine_levels(dev, oracle):
    """One segment over more than 2,600 tiles: its run of carries crosses ten
    spine CTAs (256 carries each) and is finished by the CTA it ends in; a
    segment that begins exactly on a tile edge takes the overwrite path."""
    import moderngpu_amd as m
    rng = np.random.default_rng(23)
    nv = m.segreduce_tile_size(0)
    count = 2600 * nv + 123
    values = rng.integers(-1000, 1000, size=count).astype(np.int32)
    for segs in ([0], [0, 5], [0, nv - 1], [0, nv - 1, 1030 * nv - 1030, 2000 * nv],
                 [0, 0, 0, count - 1, count, count]):
        for phases in (7, 7 | 8):       # own splits, and the partition kernel
            _check(values, np.array(segs, dtype=np.int32), "plus", -3, oracle, str(segs), phases)
            _check(values, np.array(segs, dtype=np.int32), "maximum", -3, oracle, str(segs), phases)


@pytest.mark.parametrize("tiles", [4096, 4097])
def test_either_side_of_the_partition_kernel(dev, oracle, tiles):
    """Calls of up to 4,096 tiles let every tile find its own splits; one tile
    more and the partition kernel runs.  Same input but for one value."""
    import moderngpu_amd as m
    rng = np.random.default_rng(31)
    nv = m.segreduce_tile_size(0)
    nseg = 300_000
    count = tiles * nv - nseg - nv + 1          # count + nseg = (tiles - 1) * nv + 1
    assert (count + nseg + nv - 1) // nv == tiles
    segs = random_segments(rng, count, nseg)
    values = rng.integers(-1000, 1000, size=count).astype(np.int32)
    _check(values, segs, "plus", 7, oracle, "tiles=%d" % tiles)
    _check(values.astype(np.float32), segs, "maximum", -1.0, oracle, "tiles=%d" % tiles)


def test_full_size_config2_properties(dev):
    """2^26 fp32 items: compared on the device with torch.segment_reduce
    (independent code) in float64, tolerance 1e-5 * sum|x|."""
    import torch
    import moderngpu_amd as m
    from moderngpu_amd import workloads
    w = workloads.config2()
    values, segs = _dev(w["values"]), _dev(w["segments"])
    got = m.segreduce(values, segs, "plus", 0.0)
    lens = torch.diff(torch.cat([segs.long(), torch.tensor([values.numel()], device=dev)]))
    want = torch.segment_reduce(values.double(), "sum", lengths=lens, unsafe=True)
    assert torch.all((got.double() - want).abs() <= 1e-5 * want.abs() + 1e-30)
    assert torch.all(got[lens == 0] == 0)


@pytest.mark.parametrize("kind", ["f64max", "i64sum"])
def test_full_size_config5_properties(dev, kind):
    import torch
    import moderngpu_amd as m
    from moderngpu_amd import workloads
    w = workloads.config5(kind=kind)
    values, segs = _dev(w["values"]), _dev(w["segments"])
    got = m.segreduce(values, segs, w["op"], w["init"])
    lens = torch.diff(torch.cat([segs.long(), torch.tensor([values.numel()], device=dev)]))
    if kind == "i64sum":
        # torch has no int64 segment_reduce: difference of wrapping prefix sums.
        prefix = torch.cat([torch.zeros(1, dtype=torch.int64, device=dev),
                            torch.cumsum(values, 0)])
        ends = segs.long() + lens
        want = prefix[ends] - prefix[segs.long()]
        assert torch.equal(got, want)
        assert int(got.sum().item()) == int(values.sum().item())
    else:
        want = torch.segment_reduce(values, "max", lengths=lens, unsafe=True)
        nz = lens > 0
        assert torch.equal(got[nz], want[nz])
        assert torch.all(torch.isinf(got[~nz]) & (got[~nz] < 0))


def test_lbs_segreduce_seg_plus_rank(oracle, dev):
    """lbs_segreduce through the C ABI with the reference test's functor
    (seg + rank, plus, init -1) on the layouts that stress tile boundaries."""
    import moderngpu_amd as m
    from moderngpu_amd import workloads
    from util import segment_layouts
    rng = np.random.default_rng(21)
    nv = m.segreduce_tile_size(0)
    for name, count, segs in segment_layouts(rng, nv):
        got = m.lbs_segreduce_seg_plus_rank(count, _dev(segs), init=-1)
        want = oracle.lbs_segreduce_seg_plus_rank(count, segs, init=-1)
        assert np.array_equal(got.cpu().numpy(), want), name
    for count, nseg, seed in ((10_000_000, 100, 0), (3_000_000, 100_000, 1), (40_000, 90_000, 2)):
        segs = workloads.reference_test_segments(count, nseg, seed)
        got = m.lbs_segreduce_seg_plus_rank(count, _dev(segs), init=-1)
        want = oracle.lbs_segreduce_seg_plus_rank(count, segs, init=-1)
        assert np.array_equal(got.cpu().numpy(), want), (count, nseg)


def test_prepared_calls_match_direct_calls(oracle, dev):
    """prepare_segreduce / prepare_load_balance_search marshal the arguments
    once; what they enqueue must be the ordinary call."""
    import torch
    import moderngpu_amd as m
    from moderngpu_amd import workloads
    w = workloads.config1(count=300_000, num_segments=4_000)
    values, segs = torch.from_numpy(w["values"]).to(dev), torch.from_numpy(w["segments"]).to(dev)
    call, out = m.prepare_segreduce(values, segs, "plus", 0)
    for _ in range(3):
        out.fill_(-7)
        assert call() is out
        torch.cuda.synchronize()
        assert np.array_equal(out.cpu().numpy(),
                              oracle.segreduce(w["values"], w["segments"], "plus", 0))
    call, out = m.prepare_load_balance_search(300_000, segs)
    call()
    torch.cuda.synchronize()
    assert np.array_equal(out.cpu().numpy(),
                          oracle.load_balance_search(300_000, w["segments"]))
