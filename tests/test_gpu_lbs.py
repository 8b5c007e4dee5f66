"""Partition kernels, load-balancing search, transform_lbs and the interval
functions through the C ABI, against the CPU oracle (bit-exact)."""
import json
import os

import numpy as np
import pytest

from util import lengths_of, random_segments, segment_layouts

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


def _dev(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def test_partitions_golden_and_oracle(dev, oracle):
    import moderngpu_amd as m
    g = json.load(open(os.path.join(GOLDEN, "reference_host_functions.json")))
    segs = np.array(g["segments"], dtype=np.int32)
    got = m.load_balance_partitions(g["count"], _dev(segs), 1).cpu().numpy()
    assert list(got) == g["merge_path_upper_by_diag"]

    rng = np.random.default_rng(11)
    for _ in range(12):
        count = int(rng.integers(0, 200000))
        segs = random_segments(rng, count, int(rng.integers(1, 30000)))
        spacing = int(rng.choice([1, 7, 128, 896, 4096]))
        got = m.load_balance_partitions(count, _dev(segs), spacing).cpu().numpy()
        assert np.array_equal(got, oracle.lbs_partitions(count, segs, spacing))


def test_block_partitions(dev, oracle):
    """The coarse partition the search kernels use: for every tile boundary the
    block of lbs_block starts that holds its split, i.e. (starts in front of
    the boundary - 1) // lbs_block, against the oracle's exact splits."""
    import ctypes
    import torch
    tk = ctypes.CDLL(os.path.join(os.path.dirname(__file__), "csrc", "libmgpu_test_kernels.so"))
    block = tk.tk_lbs_block()
    rng = np.random.default_rng(21)
    cases = []
    for _ in range(10):
        count = int(rng.integers(0, 400000))
        cases.append((count, random_segments(rng, count, int(rng.integers(1, 60000))),
                      int(rng.choice([64, 448, 4032, 8128]))))
    # one segment spanning very many tiles; many empty segments; one start
    cases.append((3_000_000, np.array([0, 5, 2_999_990], np.int32), 448))
    cases.append((100, np.zeros(5000, np.int32), 64))
    cases.append((77, np.array([0], np.int32), 64))
    for count, segs, spacing in cases:
        total = count + segs.size
        n = (total + spacing - 1) // spacing + 1
        got = torch.full((n,), -7, dtype=torch.int32, device="cuda")
        d_segs = _dev(segs)
        assert tk.tk_lbs_block_partitions(count, ctypes.c_void_p(d_segs.data_ptr()), segs.size,
                                          spacing, ctypes.c_void_p(got.data_ptr())) == 0
        mp = oracle.lbs_partitions(count, segs, spacing).astype(np.int64)
        diag = np.minimum(np.arange(n, dtype=np.int64) * spacing, total)
        in_front = diag - mp                      # starts in front of each boundary
        want = np.maximum(in_front - 1, 0) // block
        assert np.array_equal(got.cpu().numpy(), want), (count, segs.size, spacing)


def test_merge_path_and_binary_search_partitions(dev, oracle):
    import moderngpu_amd as m
    rng = np.random.default_rng(12)
    a = np.sort(rng.integers(0, 5000, size=30000)).astype(np.int32)
    b = np.sort(rng.integers(0, 5000, size=20000)).astype(np.int32)
    for bounds in ("lower", "upper"):
        for spacing in (1, 100, 1024):
            got = m.merge_path_partitions(_dev(a), a.size, _dev(b), spacing, bounds).cpu().numpy()
            want = oracle.merge_path_partitions(a, a.size, b, spacing, bounds == "upper")
            assert np.array_equal(got, want)
        got = m.binary_search_partitions(_dev(a), 5000, 37, bounds).cpu().numpy()
        assert np.array_equal(got, oracle.binary_search_partitions(a, 5000, 37, bounds == "upper"))


def test_lbs_reference_test_vector(dev):
    # tests/test_load_balance.cu:9-28 of the reference.
    import moderngpu_amd as m
    count, spacing = 200030, 100
    segs = np.arange(0, count, spacing, dtype=np.int32)
    got = m.load_balance_search(count, _dev(segs)).cpu().numpy()
    assert np.array_equal(got, np.arange(count) // spacing)


def test_lbs_layouts(dev, oracle):
    import moderngpu_amd as m
    rng = np.random.default_rng(13)
    layouts = list(segment_layouts(rng, m.lbs_search_tile_size())) + \
        list(segment_layouts(rng, m.lbs_tile_size()))
    for name, count, segs in layouts:
        want = oracle.load_balance_search(count, segs)
        # small calls find their own splits; 3 | 8 puts the partition kernel in front
        for phases in (3, 3 | 8):
            got = m.load_balance_search(count, _dev(segs), phases=phases).cpu().numpy()
            assert np.array_equal(got, want), (name, phases)
        seg, rank = m.transform_lbs(count, _dev(segs))
        wseg, wrank = oracle.transform_lbs(count, segs)
        assert np.array_equal(seg.cpu().numpy(), wseg), name
        assert np.array_equal(rank.cpu().numpy(), wrank), name


@pytest.mark.parametrize("tiles", [1536, 1537])
def test_either_side_of_the_partition_kernel(dev, oracle, tiles):
    """Calls of up to 1,536 tiles let the tile kernel find its own splits;
    one tile more and a partition kernel runs first."""
    import moderngpu_amd as m
    rng = np.random.default_rng(32)
    for spacing, expand in ((m.lbs_search_tile_size(), False), (m.lbs_tile_size(), True)):
        nseg = 700_000
        count = (tiles - 1) * spacing + 1 - nseg
        assert (count + nseg + spacing - 1) // spacing == tiles
        segs = random_segments(rng, count, nseg)
        if expand:
            vals = rng.integers(0, 2 ** 31, size=nseg).astype(np.int32)
            got = m.interval_expand(_dev(vals), count, _dev(segs)).cpu().numpy()
            assert np.array_equal(got, oracle.interval_expand(vals, count, segs))
        else:
            got = m.load_balance_search(count, _dev(segs)).cpu().numpy()
            assert np.array_equal(got, oracle.load_balance_search(count, segs))


@pytest.mark.parametrize("elem", [np.uint8, np.int16, np.int32, np.float64, "b16"])
def test_interval_expand(dev, oracle, elem):
    import torch
    import moderngpu_amd as m
    rng = np.random.default_rng(14)
    for name, count, segs in segment_layouts(rng, m.lbs_tile_size()):
        nseg = segs.size
        if elem == "b16":
            vals = rng.integers(0, 2 ** 62, size=(nseg, 2)).astype(np.int64)
            dv = _dev(vals).view(torch.complex128).reshape(nseg)
            got = m.interval_expand(dv, count, _dev(segs))
            got = got.view(torch.float64).view(torch.int64).reshape(count, 2).cpu().numpy()
            want = np.repeat(vals, lengths_of(segs, count), axis=0)
        else:
            vals = rng.integers(0, 120, size=nseg).astype(elem)
            got = m.interval_expand(_dev(vals), count, _dev(segs)).cpu().numpy()
            want = oracle.interval_expand(vals, count, segs)
            parted = m.interval_expand(_dev(vals), count, _dev(segs), phases=3 | 8)
            assert np.array_equal(parted.cpu().numpy(), want), name + "/partitioned"
        assert np.array_equal(got, want), name


def test_interval_gather_scatter_move(dev, oracle):
    import torch
    import moderngpu_amd as m
    rng = np.random.default_rng(15)
    count, nseg = 50000, 3000
    segs = random_segments(rng, count, nseg, dup=0.1)
    lens = lengths_of(segs, count)
    order = rng.permutation(nseg)
    dest = np.zeros(nseg, dtype=np.int64)
    dest[order] = np.concatenate([[0], np.cumsum(lens[order])[:-1]])
    dest = dest.astype(np.int32)
    src = rng.integers(0, 10 ** 6, size=count).astype(np.int32)
    got = m.interval_gather(_dev(src), count, _dev(segs), _dev(dest)).cpu().numpy()
    assert np.array_equal(got, oracle.interval_gather(src, count, segs, dest))
    out = torch.zeros(count, dtype=torch.int32, device=dev)
    m.interval_scatter(_dev(src), count, _dev(segs), _dev(dest), out)
    assert np.array_equal(out.cpu().numpy(), oracle.interval_scatter(src, count, segs, dest, count))
    gather = dest[rng.permutation(nseg)].copy()
    gather[gather.astype(np.int64) + lens > count] = 0
    out = torch.zeros(count, dtype=torch.int32, device=dev)
    m.interval_move(_dev(src), count, _dev(segs), _dev(dest), _dev(gather), out)
    assert np.array_equal(out.cpu().numpy(),
                          oracle.interval_move(src, count, segs, dest, gather, count))


def test_config3_scaled_against_oracle(dev, oracle):
    import moderngpu_amd as m
    from moderngpu_amd import workloads
    w = workloads.config3(scale=32)
    got = m.load_balance_search(w["count"], _dev(w["segments"])).cpu().numpy()
    assert np.array_equal(got, oracle.load_balance_search(w["count"], w["segments"]))
    got = m.interval_expand(_dev(w["values"]), w["count"], _dev(w["segments"])).cpu().numpy()
    assert np.array_equal(got, oracle.interval_expand(w["values"], w["count"], w["segments"]))


def test_config3_full_size_properties(dev):
    """2^24 segments / 2^28 items: checked on the device with torch ops that do
    not share code with the kernels (searchsorted closed form, repeat)."""
    import torch
    import moderngpu_amd as m
    from moderngpu_amd import workloads
    w = workloads.config3()
    count = w["count"]
    segs = _dev(w["segments"])
    got = m.load_balance_search(count, segs)
    torch.cuda.synchronize()
    step = 1 << 26
    for lo in range(0, count, step):
        idx = torch.arange(lo, min(lo + step, count), dtype=torch.int32, device=dev)
        want = torch.searchsorted(segs, idx, right=True) - 1
        assert torch.equal(got[lo:lo + step].long(), want)
        del idx, want
    vals = _dev(w["values"])
    exp = m.interval_expand(vals, count, segs)
    assert torch.equal(exp, vals[got.long()])


def test_memory_properties_and_store_yardstick(dev):
    """mgpu_hip_memory_properties returns what hipDeviceProp_t holds; the store
    yardstick of the test kernels writes every int of its ranges under each of
    its three tile-to-CTA mappings, with and without the read in front."""
    import ctypes
    import torch
    import moderngpu_amd as m
    clock, width = ctypes.c_int(0), ctypes.c_int(0)
    assert m.lib().mgpu_hip_memory_properties(0, ctypes.addressof(clock),
                                              ctypes.addressof(width)) == 0
    assert clock.value > 0 and width.value > 0 and width.value % 64 == 0
    assert m.lib().mgpu_hip_memory_properties(0, None, None) == 1      # hipErrorInvalidValue

    tk = ctypes.CDLL(os.path.join(os.path.dirname(__file__), "csrc", "libmgpu_test_kernels.so"))
    rng = np.random.default_rng(5)
    lengths = 32 * rng.integers(1, 300, size=333)
    begins = np.concatenate([[0], np.cumsum(lengths)]).astype(np.int32)
    n, tiles = int(begins[-1]), lengths.size
    d_begins = _dev(begins)
    source = torch.arange(512 * tiles, dtype=torch.int32, device="cuda")
    pos = np.arange(n) - np.repeat(begins[:-1], lengths)
    tile_of = np.repeat(np.arange(tiles), lengths)
    for mapping in (0, 1, 2):
        for read_ints in (0, 64, 512):
            out = torch.full((n + 8,), -1, dtype=torch.int32, device="cuda")
            assert tk.tk_store_probe(ctypes.c_void_p(out.data_ptr()),
                                     ctypes.c_void_p(d_begins.data_ptr()), tiles, mapping,
                                     read_ints, ctypes.c_void_p(source.data_ptr()), None) == 0
            torch.cuda.synchronize()
            got = out.cpu().numpy()
            assert (got[n:] == -1).all()
            # groups of four: position in the tile, x, 2, 3, where x is what the
            # thread's right-hand neighbour read (0 beyond read_ints)
            thread = (pos // 4) % 512
            neighbour = (thread + 1) % 512
            x = np.where(neighbour < read_ints, read_ints * tile_of + neighbour, 0)
            want = np.select([pos % 4 == 0, pos % 4 == 1], [pos, x], pos % 4)
            assert np.array_equal(got[:n], want), (mapping, read_ints)
