#!/usr/bin/env python3
"""Benchmark of the segmented-reduce / load-balancing-search path on one
MI355X.

One "step" is one complete call of the hot path (partition kernel, tile
kernel, carry spine) on a batch that is already resident in HBM.  The default
workload is BASELINE.json's configs[1]: segmented fp32 sum over 2^26 values in
2^20 geometric-length segments.  Inputs rotate over several independent copies
so that the 256 MB memory-side cache cannot serve a 256 MiB input.

Prints ONE JSON line (see the keys at the bottom).
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0      # MI355X HBM3E, published


def _dev(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


_last_config = {}


def _config(name, **kwargs):
    """workloads.<name>(**kwargs), keeping the most recent result: workloads
    measured one after the other on the same configuration generate it once."""
    from moderngpu_amd import workloads
    key = (name, tuple(sorted(kwargs.items())))
    if key not in _last_config:
        _last_config.clear()
        _last_config[key] = getattr(workloads, name)(**kwargs)
    return _last_config[key]


class Workload:
    """name, algorithmic bytes/items per step, device copies, step(i),
    tiles(i) (dominant kernel only), parity check and CPU baseline."""


def make_c2(copies):
    import torch
    import moderngpu_amd as m
    from moderngpu_amd import workloads
    w = workloads.config2()
    n, s = w["values"].size, w["segments"].size
    segs = [_dev(w["segments"]) for _ in range(copies)]
    vals = [_dev(w["values"])]
    for c in range(1, copies):          # independent values per copy
        vals.append(torch.rand(n, dtype=torch.float32, device="cuda"))
    outs = [torch.empty(s, dtype=torch.float32, device="cuda") for _ in range(copies)]
    wk = Workload()
    wk.name = "segreduce fp32 plus, 2^26 values, 2^20 geometric segments (mean 64, ~5% empty)"
    wk.key = "c2_segreduce_f32"
    wk.dtype = "f32"
    wk.items = n
    wk.bytes = n * 4 + s * 4 + s * 4
    wk.kernel = "segreduce_tile_f<256x16, float, plus>"
    # Arguments are marshalled once per copy: a step is the C call alone, as it
    # is for a C or C++ caller.
    calls = [m.prepare_segreduce(vals[c], segs[c], "plus", 0.0, out=outs[c])[0]
             for c in range(copies)]
    tiles = [m.prepare_segreduce(vals[c], segs[c], "plus", 0.0, out=outs[c], phases=2)[0]
             for c in range(copies)]
    wk.step = lambda i: calls[i % copies]()
    wk.tiles = lambda i: tiles[i % copies]()

    def check():
        got = m.segreduce(vals[0], segs[0], "plus", 0.0, out=outs[0])
        lens = torch.diff(torch.cat([segs[0].long(), torch.tensor([n], device="cuda")]))
        want = torch.segment_reduce(vals[0].double(), "sum", lengths=lens, unsafe=True)
        ok = torch.all((got.double() - want).abs() <= 1e-5 * want.abs() + 1e-30)
        # and a slice against the CPU oracle itself
        from oracle import oracle
        k = 1 << 14
        cnt = int(w["segments"][k])
        ref = oracle.segreduce(w["values"][:cnt], w["segments"][:k], "plus", 0.0)
        ok2 = np.all(np.abs(got[:k - 1].cpu().numpy() - ref[:k - 1]) <=
                     1e-5 * np.abs(ref[:k - 1]))
        return bool(ok) and bool(ok2)
    wk.check = check

    def cpu():
        from oracle import oracle
        return lambda: oracle.segreduce(w["values"], w["segments"], "plus", 0.0)
    wk.cpu = cpu

    def cpu_threads(threads):
        from oracle import oracle
        return lambda: oracle.segreduce_threads(w["values"], w["segments"], "plus", 0.0,
                                                threads=threads)
    wk.cpu_threads = cpu_threads
    return wk


def make_c3(copies, expand=False):
    import torch
    import moderngpu_amd as m
    w = _config("config3")
    n, s = w["count"], w["segments"].size
    segs = [_dev(w["segments"]) for _ in range(copies)]
    vals = [_dev(w["values"]) for _ in range(copies)]
    outs = [torch.empty(n, dtype=torch.int32, device="cuda") for _ in range(copies)]
    wk = Workload()
    wk.dtype = "i32"
    wk.items = n
    if expand:
        wk.key = "c3_interval_expand_i32"
        wk.name = "interval_expand int32, 2^24 Zipf(1.2) segments, 2^28 items"
        wk.bytes = s * 4 + s * 4 + n * 4
        wk.kernel = "transform_lbs_f<512x16, expand>"
        wk.step = lambda i: m.interval_expand(vals[i % copies], n, segs[i % copies],
                                              out=outs[i % copies])
        wk.tiles = lambda i: m.interval_expand(vals[i % copies], n, segs[i % copies],
                                               out=outs[i % copies], phases=2)
    else:
        wk.key = "c3_load_balance_search"
        wk.name = "load_balance_search, 2^24 Zipf(1.2) segments, 2^28 items"
        wk.bytes = s * 4 + n * 4
        wk.kernel = "transform_lbs_f<512x16, store seg>"
        calls = [m.prepare_load_balance_search(n, segs[c], out=outs[c])[0]
                 for c in range(copies)]
        tiles = [m.prepare_load_balance_search(n, segs[c], out=outs[c], phases=2)[0]
                 for c in range(copies)]
        wk.step = lambda i: calls[i % copies]()
        wk.tiles = lambda i: tiles[i % copies]()

    def check():
        got = wk.step(0)
        torch.cuda.synchronize()
        step = 1 << 26
        for lo in range(0, n, step):
            idx = torch.arange(lo, min(lo + step, n), dtype=torch.int32, device="cuda")
            want = torch.searchsorted(segs[0], idx, right=True) - 1
            if expand:
                want = vals[0][want]
                if not torch.equal(got[lo:lo + step], want):
                    return False
            elif not torch.equal(got[lo:lo + step].long(), want):
                return False
        return True
    wk.check = check

    def cpu():
        from oracle import oracle
        if expand:
            return lambda: oracle.interval_expand(w["values"], n, w["segments"])
        return lambda: oracle.load_balance_search(n, w["segments"])
    wk.cpu = cpu
    return wk


def make_c3_moves(copies, kind):
    """interval_gather / interval_scatter / interval_move on the C3 segments:
    every segment's items live, on the gathered or scattered side, at a
    random place of their own (the segments laid out in a random order)."""
    import torch
    import moderngpu_amd as m
    from moderngpu_amd import workloads
    from oracle import oracle
    copies = min(copies, 2)
    w = workloads.config3()
    n, s = w["count"], w["segments"].size
    lengths = np.diff(np.append(w["segments"].astype(np.int64), n))
    order = np.random.Generator(np.random.PCG64(43)).permutation(s)
    base = np.zeros(s, dtype=np.int64)
    base[order] = np.cumsum(lengths[order]) - lengths[order]
    base = base.astype(np.int32)
    segs = [_dev(w["segments"]) for _ in range(copies)]
    bases = [_dev(base) for _ in range(copies)]
    inp_host = np.random.Generator(np.random.PCG64(44)).integers(
        0, 2 ** 31, size=n, dtype=np.int64).astype(np.int32)
    inps = [_dev(inp_host) for _ in range(copies)]
    outs = [torch.empty(n, dtype=torch.int32, device="cuda") for _ in range(copies)]
    wk = Workload()
    wk.dtype, wk.items = "i32", n
    wk.key = "c3_interval_%s_i32" % kind
    wk.name = "interval_%s int32, 2^24 Zipf(1.2) segments, 2^28 items, segments placed " \
              "in random order" % kind
    wk.kernel = "partition + transform_lbs_f<512x16, %s>" % kind
    wk.bytes = n * 4 + n * 4 + s * 4 + s * 4 * (2 if kind == "move" else 1)
    if kind == "gather":
        wk.step = lambda i: m.interval_gather(inps[i % copies], n, segs[i % copies],
                                              bases[i % copies], out=outs[i % copies])
        want = lambda: oracle.interval_gather(inp_host, n, w["segments"], base)
    elif kind == "scatter":
        wk.step = lambda i: m.interval_scatter(inps[i % copies], n, segs[i % copies],
                                               bases[i % copies], outs[i % copies])
        want = lambda: oracle.interval_scatter(inp_host, n, w["segments"], base, n)
    else:
        # move = gather from the random layout back to segment order
        wk.step = lambda i: m.interval_move(inps[i % copies], n, segs[i % copies],
                                            segs[i % copies], bases[i % copies],
                                            outs[i % copies])
        want = lambda: oracle.interval_move(inp_host, n, w["segments"], w["segments"],
                                            base, n)
    wk.tiles = wk.step
    wk.check = lambda: bool(np.array_equal(wk.step(0).cpu().numpy(), want()))
    wk.cpu = lambda: want
    return wk


def make_lbs_segreduce(copies):
    """lbs_segreduce with the reference test's functor (seg + rank) on the C2
    segments: the items are computed, so the only traffic is the starts in
    and one sum per segment out."""
    import torch
    import moderngpu_amd as m
    from moderngpu_amd import workloads
    from oracle import oracle
    w = workloads.config2()
    n, s = w["values"].size, w["segments"].size
    segs = [_dev(w["segments"]) for _ in range(copies)]
    outs = [torch.empty(s, dtype=torch.int32, device="cuda") for _ in range(copies)]
    wk = Workload()
    wk.dtype, wk.items = "i32", n
    wk.key = "c2_lbs_segreduce_i32"
    wk.name = "lbs_segreduce f = seg + rank, int32 plus, 2^26 computed items, 2^20 segments"
    wk.kernel = "partition + segreduce_tile_f<lbs input> + spine"
    wk.bytes = s * 4 + s * 4
    wk.step = lambda i: m.lbs_segreduce_seg_plus_rank(n, segs[i % copies], -1,
                                                      out=outs[i % copies])
    wk.tiles = wk.step
    wk.check = lambda: bool(np.array_equal(
        wk.step(0).cpu().numpy(), oracle.lbs_segreduce_seg_plus_rank(n, w["segments"], -1)))
    wk.cpu = lambda: (lambda: oracle.lbs_segreduce_seg_plus_rank(n, w["segments"], -1))
    return wk


def make_search(copies, kind):
    """sorted_search: 2^26 sorted needles in 2^26 sorted haystack keys, both
    uniform in [0, 2^28).  inner_join: 2^24 keys a side, uniform in [0, 2^24)
    (about one match per key)."""
    import torch
    import moderngpu_amd as m
    from oracle import oracle
    rng = np.random.Generator(np.random.PCG64(42))
    wk = Workload()
    wk.dtype = "i32"
    if kind == "search":
        n = h = 1 << 26
        needles = np.sort(rng.integers(0, 1 << 28, size=n, dtype=np.int32))
        haystack = np.sort(rng.integers(0, 1 << 28, size=h, dtype=np.int32))
        dn = [_dev(needles) for _ in range(copies)]
        dh = [_dev(haystack) for _ in range(copies)]
        outs = [torch.empty(n, dtype=torch.int32, device="cuda") for _ in range(copies)]
        wk.key, wk.items = "sorted_search_i32", n
        wk.name = "sorted_search lower bound, 2^26 needles in 2^26 haystack keys"
        wk.bytes = n * 4 + h * 4 + n * 4
        wk.kernel = "partition + sorted_search_f<256x12>"
        wk.step = lambda i: m.sorted_search(dn[i % copies], dh[i % copies], "lower",
                                            out=outs[i % copies])
        wk.check = lambda: bool(np.array_equal(
            wk.step(0).cpu().numpy(), np.searchsorted(haystack, needles, side="left")))
        wk.cpu = lambda: (lambda: oracle.sorted_search(needles, haystack))
    else:
        n = 1 << 24
        a = np.sort(rng.integers(0, n, size=n, dtype=np.int32))
        b = np.sort(rng.integers(0, n, size=n, dtype=np.int32))
        da = [_dev(a) for _ in range(copies)]
        db = [_dev(b) for _ in range(copies)]
        pairs = int(oracle.inner_join(a, b).shape[0])
        wk.key, wk.items = "inner_join_i32", 2 * n
        wk.name = "inner_join, 2^24 keys a side, %d pairs" % pairs
        wk.bytes = 2 * n * 4 + pairs * 8
        wk.kernel = "sorted_search (lower + counts) + scan + transform_lbs"
        wk.step = lambda i: m.inner_join(da[i % copies], db[i % copies])
        wk.check = lambda: bool(np.array_equal(wk.step(0).cpu().numpy(),
                                               oracle.inner_join(a, b)))
        wk.cpu = lambda: (lambda: oracle.inner_join(a, b))
    wk.tiles = wk.step
    return wk


def make_c4(copies):
    import torch
    import moderngpu_amd as m
    w = _config("config4")
    nnz, rows = w["nnz"], w["segments"].size
    mats = [_dev(w["matrix"]) for _ in range(copies)]
    cols = [_dev(w["columns"]) for _ in range(copies)]
    segs = [_dev(w["segments"]) for _ in range(copies)]
    x = _dev(w["vector"])
    outs = [torch.empty(rows, dtype=torch.float32, device="cuda") for _ in range(copies)]
    wk = Workload()
    wk.key = "c4_spmv_f32"
    wk.name = "spmv fp32, 2^22 rows, Zipf(1.5) row lengths (mean 16), %d nonzeros" % nnz
    wk.dtype = "f32"
    wk.items = nnz
    wk.bytes = nnz * 8 + rows * 4 + rows * 4 + rows * 4
    wk.kernel = "segreduce_tile_f<256x16, spmv float>"
    wk.step = lambda i: m.spmv(mats[i % copies], cols[i % copies], x, segs[i % copies],
                               out=outs[i % copies])
    wk.tiles = lambda i: m.spmv(mats[i % copies], cols[i % copies], x, segs[i % copies],
                                out=outs[i % copies], phases=2)

    def check():
        got = wk.step(0)
        lens = torch.diff(torch.cat([segs[0].long(), torch.tensor([nnz], device="cuda")]))
        prod = mats[0].double() * x.double()[cols[0].long()]
        want = torch.segment_reduce(prod, "sum", lengths=lens, unsafe=True)
        norm = torch.segment_reduce(prod.abs(), "sum", lengths=lens, unsafe=True)
        return bool(torch.all((got.double() - want).abs() <= 1e-5 * norm + 1e-30))
    wk.check = check

    def cpu():
        from oracle import oracle
        return lambda: oracle.spmv(w["matrix"], w["columns"], w["vector"], w["segments"])
    wk.cpu = cpu
    return wk


def make_c4_gather_probe(copies):
    """Not a kernel of this library: torch's index_select over the column
    indices of configs[3], y[i] = x[columns[i]] -- the same 2^26 gathers into
    the same 16 MiB vector as spmv does, and nothing else but one store per
    gather.  A yardstick for the device's gather rate."""
    import torch
    w = _config("config4")
    nnz, rows = w["nnz"], w["segments"].size
    cols = [_dev(w["columns"]) for _ in range(copies)]
    x = _dev(w["vector"])
    outs = [torch.empty(nnz, dtype=torch.float32, device="cuda") for _ in range(copies)]
    wk = Workload()
    wk.key, wk.dtype, wk.items = "c4_gather_probe_f32", "f32", nnz
    wk.name = "torch.index_select(x, columns): %d gathers into 2^22 floats" % nnz
    wk.bytes = nnz * 4 + nnz * 4 + rows * 4
    wk.kernel = "torch index_select (yardstick, not part of the library)"
    wk.step = lambda i: torch.index_select(x, 0, cols[i % copies], out=outs[i % copies])
    wk.tiles = wk.step
    wk.check = lambda: bool(np.array_equal(wk.step(0).cpu().numpy(),
                                           w["vector"][w["columns"]]))
    wk.cpu = lambda: (lambda: w["vector"][w["columns"]])
    return wk


def make_store_probe(copies, mapping, read_ints):
    """Not a kernel of this library: the yardstick for the kernels that are
    streams of stores (tests/csrc/test_kernels.hip, tk_store_probe).  1 GiB of
    ints is written by CTAs of 512 threads, each one range of about 7,650 ints
    whose ends are multiples of 32 (what a tile of the search stores); before
    that each CTA reads read_ints ints of its own from a second array.
    mapping: 0 tile = blockIdx, 1 runs of 16 tiles per XCD, 2 eighths."""
    import ctypes
    import torch
    tk = ctypes.CDLL(os.path.join(ROOT, "tests", "csrc", "libmgpu_test_kernels.so"))
    n = 1 << 28
    rng = np.random.Generator(np.random.PCG64(1))
    ends = np.cumsum(7650 + rng.integers(-200, 201, size=n // 7650 + 8))
    ends = np.unique((ends - ends % 32)[ends < n - 8000])
    begins = np.concatenate([[0], ends, [n]]).astype(np.int32)
    tiles = begins.size - 1
    d_begins = _dev(begins)
    outs = [torch.empty(n, dtype=torch.int32, device="cuda") for _ in range(min(copies, 2))]
    source = torch.zeros(max(read_ints, 1) * tiles + 512, dtype=torch.int32, device="cuda")
    wk = Workload()
    names = ["tile = blockIdx", "runs of 16 tiles per XCD", "one eighth of the tiles per XCD"]
    wk.key = "store_probe_%s_read%d" % (["linear", "runs", "eighths"][mapping], read_ints)
    wk.dtype, wk.items = "i32", n
    wk.name = ("store yardstick: 1 GiB in %d ragged tiles, %s, %d bytes read per tile"
               % (tiles, names[mapping], 4 * read_ints))
    wk.bytes = n * 4 + read_ints * 4 * tiles
    wk.kernel = "store_probe_k (yardstick, not part of the library)"
    stream = lambda: ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)

    def step(i):
        out = outs[i % len(outs)]
        rc = tk.tk_store_probe(ctypes.c_void_p(out.data_ptr()),
                               ctypes.c_void_p(d_begins.data_ptr()), tiles, mapping, read_ints,
                               ctypes.c_void_p(source.data_ptr()), stream())
        assert rc == 0, rc
        return out
    wk.step = wk.tiles = step

    def check():
        # Every tile is a whole number of groups of four: q, x, 2, 3 with q the
        # position in the tile and x = 0 (the source array is all zeros).
        got = step(0)
        b = d_begins.long()
        first = torch.arange(n, device="cuda") - torch.repeat_interleave(b[:-1], b[1:] - b[:-1])
        m = first % 4
        want = torch.where(m == 0, first, torch.where(m == 1, torch.zeros_like(m), m)).int()
        return bool(torch.equal(got, want))
    wk.check = check
    wk.cpu = lambda: (lambda: np.zeros(n, dtype=np.int32))
    return wk


def make_c5(copies, kind):
    import torch
    import moderngpu_amd as m
    from moderngpu_amd import workloads
    w = workloads.config5(kind=kind)
    n, s = w["values"].size, w["segments"].size
    vals = [_dev(w["values"]) for _ in range(copies)]
    segs = [_dev(w["segments"]) for _ in range(copies)]
    outs = [torch.empty(s, dtype=vals[0].dtype, device="cuda") for _ in range(copies)]
    wk = Workload()
    wk.key = "c5_" + kind
    wk.name = "segreduce %s, 2^27 values, 2^18 segments, four of ~2^25 items" % kind
    wk.dtype = "f64" if kind == "f64max" else "i64"
    wk.items = n
    wk.bytes = n * 8 + s * 4 + s * 8
    wk.kernel = "segreduce_tile_f<128x16, %s>" % kind
    calls = [m.prepare_segreduce(vals[c], segs[c], w["op"], w["init"], out=outs[c])[0]
             for c in range(copies)]
    tiles = [m.prepare_segreduce(vals[c], segs[c], w["op"], w["init"], out=outs[c],
                                 phases=2)[0] for c in range(copies)]
    wk.step = lambda i: calls[i % copies]()
    wk.tiles = lambda i: tiles[i % copies]()

    def check():
        got = wk.step(0)
        lens = torch.diff(torch.cat([segs[0].long(), torch.tensor([n], device="cuda")]))
        nz = lens > 0
        if kind == "f64max":
            want = torch.segment_reduce(vals[0], "max", lengths=lens, unsafe=True)
        else:       # wrapping prefix sums (torch has no int64 segment_reduce)
            prefix = torch.cat([torch.zeros(1, dtype=torch.int64, device="cuda"),
                                torch.cumsum(vals[0], 0)])
            want = prefix[segs[0].long() + lens] - prefix[segs[0].long()]
        return bool(torch.equal(got[nz], want[nz]))
    wk.check = check

    def cpu():
        from oracle import oracle
        return lambda: oracle.segreduce(w["values"], w["segments"], w["op"], w["init"])
    wk.cpu = cpu

    def cpu_threads(threads):
        from oracle import oracle
        return lambda: oracle.segreduce_threads(w["values"], w["segments"], w["op"],
                                                w["init"], threads=threads)
    wk.cpu_threads = cpu_threads
    return wk


def make_c2_typed(copies, dtype_name, op):
    """segreduce on the C2 segments for any of the library's value types and
    operators (the headline workload is float32 plus): integer results must
    equal the CPU loop's, floating ones must lie within 1e-5 (float32) or 1e-12
    (float64) of it, relative to the sum of the segment's magnitudes."""
    import torch
    import moderngpu_amd as m
    from moderngpu_amd import workloads
    from oracle import oracle
    np_type = {"i32": np.int32, "u32": np.uint32, "f32": np.float32,
               "i64": np.int64, "u64": np.uint64, "f64": np.float64}[dtype_name]
    unsigned = dtype_name in ("u32", "u64")
    copies = min(copies, 3)
    count, starts = workloads.config2_segments()
    s = starts.size
    rng = np.random.Generator(np.random.PCG64(7))
    if np.dtype(np_type).kind == "f":
        host = [rng.random(count, dtype=np_type) for _ in range(copies)]
    else:
        host = [rng.integers(0, 1 << 20, size=count, dtype=np.int64).astype(np_type)
                for _ in range(copies)]
    as_signed = {np.uint32: np.int32, np.uint64: np.int64}
    vals = [_dev(h.view(as_signed[np_type]) if unsigned else h) for h in host]
    segs = [_dev(starts) for _ in range(copies)]
    outs = [torch.empty(s, dtype=vals[0].dtype, device="cuda") for _ in range(copies)]
    size = host[0].itemsize
    wk = Workload()
    wk.key = "c2_segreduce_%s_%s" % (dtype_name, op)
    wk.name = "segreduce %s %s, 2^26 values, 2^20 geometric segments" % (dtype_name, op)
    wk.dtype, wk.items = dtype_name, count
    wk.bytes = count * size + s * 4 + s * size
    wk.kernel = "segreduce_tile_f<%s, %s>" % (dtype_name, op)
    calls = [m.prepare_segreduce(vals[c], segs[c], op, 0, out=outs[c], unsigned=unsigned)[0]
             for c in range(copies)]
    tiles = [m.prepare_segreduce(vals[c], segs[c], op, 0, out=outs[c], unsigned=unsigned,
                                 phases=2)[0] for c in range(copies)]
    wk.step = lambda i: calls[i % copies]()
    wk.tiles = lambda i: tiles[i % copies]()

    def check():
        got = calls[0]().cpu().numpy()
        got = got.view(np_type) if unsigned else got
        want = oracle.segreduce(host[0], starts, op, 0)
        if np.dtype(np_type).kind != "f":
            return bool(np.array_equal(got, want))
        tol = 1e-5 if np_type == np.float32 else 1e-12
        # the values are not negative: |want| is the sum of magnitudes
        return bool(np.all(np.abs(got.astype(np.float64) - want.astype(np.float64))
                           <= tol * np.abs(want) + 1e-300))
    wk.check = check
    wk.cpu = lambda: (lambda: oracle.segreduce(host[0], starts, op, 0))
    return wk


def make_shape(copies, spec):
    """Workloads of a given shape, for looking at the library outside the
    BASELINE configurations: --workload shape:<op>:<log2 items>:<segments>
      op        segreduce (float32 plus) | lbs (load_balance_search) |
                expand<bytes> (interval_expand of 1/2/4/8/16-byte elements) |
                gather<bytes>, scatter<bytes>, move<bytes> (the interval moves
                with every segment in place)
      segments  len<k>   every segment k items long
                nseg<k>  k segments, starts drawn uniformly (sorted)
    e.g. shape:segreduce:26:nseg1024, shape:lbs:20:len16, shape:expand16:28:len16.
    Parity: segreduce against float64 sums (1e-5 of the sum of magnitudes), lbs
    and expand against numpy."""
    import torch
    import moderngpu_amd as m
    from oracle import oracle
    _, op, log2n, segspec = spec.split(":")
    n = 1 << int(log2n)
    rng = np.random.Generator(np.random.PCG64(11))
    if segspec.startswith("len"):
        starts = np.arange(0, n, int(segspec[3:]), dtype=np.int64)
    elif segspec.startswith("nseg"):
        k = int(segspec[4:])
        starts = np.concatenate([[0], np.sort(rng.integers(0, n, size=k - 1))])
    else:
        raise ValueError("segments: len<k> or nseg<k>")
    starts = starts.astype(np.int32)
    s = starts.size
    copies = min(copies, 3)
    segs = _dev(starts)
    wk = Workload()
    wk.key, wk.items = spec, n
    wk.kernel = "whole call"
    if op == "segreduce":
        host = [rng.random(n, dtype=np.float32) for _ in range(copies)]
        vals = [_dev(h) for h in host]
        out = torch.empty(s, dtype=torch.float32, device="cuda")
        calls = [m.prepare_segreduce(v, segs, "plus", 0.0, out=out)[0] for v in vals]
        tiles = [m.prepare_segreduce(v, segs, "plus", 0.0, out=out, phases=2)[0] for v in vals]
        wk.dtype, wk.bytes = "f32", n * 4 + s * 4 + s * 4
        wk.name = "segreduce float32 plus, 2^%s values, %d segments (%s)" % (log2n, s, segspec)
        wk.step = lambda i: calls[i % copies]()
        wk.tiles = lambda i: tiles[i % copies]()
        wk.kernel = "segreduce_tile_f<256x16, float, plus>"

        def check():
            # float64 sums of the same values (they are not negative, so the
            # sum is also the sum of magnitudes the tolerance is relative to)
            got = calls[0]().cpu().numpy().astype(np.float64)
            c = np.concatenate([[0.0], np.cumsum(host[0], dtype=np.float64)])
            ends = np.append(starts[1:], n).astype(np.int64)
            want = c[ends] - c[starts.astype(np.int64)]
            return bool(np.all(np.abs(got - want) <= 1e-5 * np.abs(want) + 1e-30))
        wk.check = check
        wk.cpu = lambda: (lambda: oracle.segreduce(host[0], starts, "plus", 0.0))
    elif op == "lbs":
        outs = [torch.empty(n, dtype=torch.int32, device="cuda") for _ in range(copies)]
        calls = [m.prepare_load_balance_search(n, segs, out=o)[0] for o in outs]
        wk.dtype, wk.bytes = "i32", n * 4 + s * 4
        wk.name = "load_balance_search, 2^%s items, %d segments (%s)" % (log2n, s, segspec)
        wk.step = lambda i: calls[i % copies]()
        wk.tiles = wk.step
        want = lambda: (np.searchsorted(starts, np.arange(n, dtype=np.int32), side="right")
                        - 1).astype(np.int32)
        wk.check = lambda: bool(np.array_equal(wk.step(0).cpu().numpy(), want()))
        wk.cpu = lambda: (lambda: oracle.load_balance_search(n, starts))
    elif op.startswith("expand"):
        size = int(op[6:])
        words = max(size // 8, 1)
        np_type = {1: np.uint8, 2: np.int16, 4: np.int32}.get(size, np.int64)
        host = rng.integers(0, 100, size=(s, words) if size == 16 else s).astype(np_type)
        vals = _dev(host)
        if size == 16:
            vals = vals.view(torch.complex128).reshape(s)
        outs = [torch.empty(n, dtype=vals.dtype, device="cuda") for _ in range(min(copies, 2))]
        wk.dtype, wk.bytes = "%d-byte" % size, n * size + s * 4 + s * size
        wk.name = "interval_expand of %d-byte elements, 2^%s items, %d segments (%s)" % (
            size, log2n, s, segspec)
        wk.step = lambda i: m.interval_expand(vals, n, segs, out=outs[i % len(outs)])
        wk.tiles = wk.step

        def check():
            got = wk.step(0)
            if size == 16:
                got = got.view(torch.float64).view(torch.int64).reshape(n, 2)
            lens = np.diff(np.append(starts.astype(np.int64), n))
            return bool(np.array_equal(got.cpu().numpy(), np.repeat(host, lens, axis=0)))
        wk.check = check
        wk.cpu = lambda: (lambda: np.repeat(host, np.diff(np.append(starts.astype(np.int64), n)),
                                            axis=0))
    elif op[:6] in ("gather", "scatte") or op.startswith("move"):
        # interval_gather / _scatter / _move with every segment in place
        # (its base is its own start): the output equals the input.
        kind = "gather" if op.startswith("gather") else (
            "scatter" if op.startswith("scatter") else "move")
        size = int(op[len(kind):])
        host = rng.integers(0, 1 << 30, size=(n, 2) if size == 16 else n).astype(
            {1: np.uint8, 2: np.int16, 4: np.int32}.get(size, np.int64))
        inp = _dev(host)
        if size == 16:
            inp = inp.view(torch.complex128).reshape(n)
        out = torch.empty_like(inp)
        wk.dtype, wk.bytes = "%d-byte" % size, 2 * n * size + 2 * s * 4
        wk.name = "interval_%s of %d-byte elements, 2^%s items, %d segments in place (%s)" % (
            kind, size, log2n, s, segspec)
        if kind == "gather":
            wk.step = lambda i: m.interval_gather(inp, n, segs, segs, out=out)
        elif kind == "scatter":
            wk.step = lambda i: m.interval_scatter(inp, n, segs, segs, out)
        else:
            wk.step = lambda i: m.interval_move(inp, n, segs, segs, segs, out)
        wk.tiles = wk.step
        as_ints = lambda t: t.view(torch.float64).view(torch.int64) if size == 16 else t
        wk.check = lambda: bool(torch.equal(as_ints(wk.step(0)), as_ints(inp)))
        wk.cpu = lambda: (lambda: host.copy())
    else:
        raise ValueError("op: segreduce, lbs, expand<bytes>, gather<bytes>, scatter<bytes> "
                         "or move<bytes>")
    return wk


def make_cumsum_probe(copies):
    """Not a kernel of this library: torch.cumsum over 2^26 int32, the
    single-pass scan the platform's library offers, beside scan_i32."""
    import torch
    n = 1 << 26
    rng = np.random.Generator(np.random.PCG64(42))
    host = rng.integers(0, 128, size=n, dtype=np.int32)
    xs = [_dev(host) for _ in range(copies)]
    outs = [torch.empty(n, dtype=torch.int32, device="cuda") for _ in range(copies)]
    wk = Workload()
    wk.key, wk.dtype, wk.items = "scan_probe_torch_cumsum_i32", "i32", n
    wk.name = "torch.cumsum (inclusive), 2^26 int32"
    wk.bytes = n * 4 + n * 4
    wk.kernel = "torch cumsum (yardstick, not part of the library)"
    wk.step = lambda i: torch.cumsum(xs[i % copies], 0, dtype=torch.int32, out=outs[i % copies])
    wk.tiles = wk.step
    wk.check = lambda: bool(np.array_equal(wk.step(0).cpu().numpy(),
                                           np.cumsum(host, dtype=np.int32)))
    wk.cpu = lambda: (lambda: np.cumsum(host, dtype=np.int32))
    return wk


def make_c1(copies):
    import torch
    import moderngpu_amd as m
    from moderngpu_amd import workloads
    from oracle import oracle
    w = workloads.config1()
    n, s = w["values"].size, w["segments"].size
    vals, segs = _dev(w["values"]), _dev(w["segments"])
    out = torch.empty(s, dtype=torch.int32, device="cuda")
    wk = Workload()
    wk.key = "c1_segreduce_i32"
    wk.name = "segreduce int32 plus, 10^6 values, 10^4 segments"
    wk.dtype = "i32"
    wk.items = n
    wk.bytes = n * 4 + s * 4 + s * 4
    wk.kernel = "segreduce_tile_f<256x16, int, plus>"
    # At this size the Python side of an unprepared call (argument checks,
    # ctypes conversion) costs more than the three kernels.
    call = m.prepare_segreduce(vals, segs, "plus", 0, out=out)[0]
    tiles = m.prepare_segreduce(vals, segs, "plus", 0, out=out, phases=2)[0]
    wk.step = lambda i: call()
    wk.tiles = lambda i: tiles()
    wk.check = lambda: bool(np.array_equal(
        wk.step(0).cpu().numpy(), oracle.segreduce(w["values"], w["segments"], "plus", 0)))
    wk.cpu = lambda: (lambda: oracle.segreduce(w["values"], w["segments"], "plus", 0))
    return wk


def make_scan(copies, kind):
    """The step in front of the path: 2^26 int32 segment lengths -> starts
    (exclusive plus-scan), or the fold of 2^26 floats (reduce)."""
    import torch
    import moderngpu_amd as m
    from oracle import oracle
    n = 1 << 26
    rng = np.random.Generator(np.random.PCG64(42))
    wk = Workload()
    wk.items = n
    if kind == "scan":
        host = rng.integers(0, 128, size=n, dtype=np.int32)
        vals = [_dev(host)] + [torch.randint(0, 128, (n,), dtype=torch.int32, device="cuda")
                               for _ in range(copies - 1)]
        outs = [torch.empty(n, dtype=torch.int32, device="cuda") for _ in range(copies)]
        red = torch.zeros(1, dtype=torch.int32, device="cuda")
        wk.key, wk.dtype = "scan_i32", "i32"
        wk.name = "exclusive plus-scan, 2^26 int32 (segment lengths -> starts)"
        wk.bytes = n * 4 + n * 4
        wk.kernel = "scan upsweep + spine + downsweep"
        wk.step = lambda i: m.scan(vals[i % copies], "plus", out=outs[i % copies],
                                   reduction=red)[0]
        wk.tiles = wk.step
        wk.check = lambda: bool(np.array_equal(
            wk.step(0).cpu().numpy(), oracle.scan(host, "plus", 0, inclusive=False)[0]))
        wk.cpu = lambda: (lambda: oracle.scan(host, "plus", 0, inclusive=False))
    else:
        host = rng.random(n, dtype=np.float32)
        vals = [_dev(host)] + [torch.rand(n, dtype=torch.float32, device="cuda")
                               for _ in range(copies - 1)]
        out = torch.zeros(1, dtype=torch.float32, device="cuda")
        wk.key, wk.dtype = "reduce_f32", "f32"
        wk.name = "plus-reduce, 2^26 float32"
        wk.bytes = n * 4
        wk.kernel = "scan_upsweep_f + reduce_final_f"
        wk.step = lambda i: m.reduce(vals[i % copies], "plus", out=out)
        wk.tiles = wk.step

        def check():
            got = float(wk.step(0).item())
            exact = float(np.sum(host.astype(np.float64)))
            return abs(got - exact) <= 1e-5 * exact
        wk.check = check
        wk.cpu = lambda: (lambda: oracle.scan(host, "plus", 0, inclusive=True))
    return wk


def make_workcreate(copies):
    """The step behind the path: 2^26 work-items in 2^20 segments (the segments
    of configs[1]), a quarter of them creating 1..8 new work-items each."""
    import torch
    import moderngpu_amd as m
    from moderngpu_amd import workloads
    from oracle import oracle
    w = workloads.config2()
    n, s = w["values"].size, w["segments"].size
    rng = np.random.Generator(np.random.PCG64(42))
    host = rng.integers(1, 9, size=n, dtype=np.int32)
    host[rng.random(n) >= 0.25] = 0
    created = [_dev(host) for _ in range(copies)]
    segs = [_dev(w["segments"]) for _ in range(copies)]
    k = int(np.count_nonzero(host))
    wk = Workload()
    wk.key, wk.dtype = "workcreate_i32", "i32"
    wk.name = ("lbs_workcreate upsweep + downsweep, 2^26 items in 2^20 segments, "
               "%d items create work" % k)
    wk.items = n
    # upsweep: counts + starts in; downsweep: starts + the creators' counts in,
    # four ints per new segment out.
    wk.bytes = n * 4 + s * 4 + s * 4 + k * 4 + k * 16
    wk.kernel = "workcreate upsweep + scan + downsweep"
    wk.step = lambda i: m.workcreate(created[i % copies], segs[i % copies])
    wk.tiles = wk.step

    def check():
        got = wk.step(0)
        want = oracle.workcreate(host, w["segments"])
        return got[0] == want[0] and all(
            np.array_equal(g.cpu().numpy(), x) for g, x in zip(got[1:], want[1:]))
    wk.check = check
    wk.cpu = lambda: (lambda: oracle.workcreate(host, w["segments"]))
    return wk


FACTORIES = {
    "workcreate_i32": make_workcreate,
    "scan_i32": lambda c: make_scan(c, "scan"),
    "reduce_f32": lambda c: make_scan(c, "reduce"),
    "c1_segreduce_i32": make_c1,
    "c2_segreduce_f32": make_c2,
    "c3_load_balance_search": lambda c: make_c3(c, False),
    "c3_interval_expand_i32": lambda c: make_c3(c, True),
    "c3_interval_gather_i32": lambda c: make_c3_moves(c, "gather"),
    "c3_interval_scatter_i32": lambda c: make_c3_moves(c, "scatter"),
    "c3_interval_move_i32": lambda c: make_c3_moves(c, "move"),
    "c2_lbs_segreduce_i32": make_lbs_segreduce,
    "sorted_search_i32": lambda c: make_search(c, "search"),
    "inner_join_i32": lambda c: make_search(c, "join"),
    "c4_spmv_f32": make_c4,
    "c4_gather_probe_f32": make_c4_gather_probe,
    "scan_probe_torch_cumsum_i32": make_cumsum_probe,
    "store_probe_linear_read0": lambda c: make_store_probe(c, 0, 0),
    "store_probe_runs_read0": lambda c: make_store_probe(c, 1, 0),
    "store_probe_eighths_read0": lambda c: make_store_probe(c, 2, 0),
    "store_probe_linear_read512": lambda c: make_store_probe(c, 0, 512),
    "store_probe_runs_read512": lambda c: make_store_probe(c, 1, 512),
    "store_probe_eighths_read512": lambda c: make_store_probe(c, 2, 512),
    "store_probe_eighths_read64": lambda c: make_store_probe(c, 2, 64),
    "c5_f64max": lambda c: make_c5(c, "f64max"),
    "c5_i64sum": lambda c: make_c5(c, "i64sum"),
}

for _t in ("i32", "u32", "f32", "i64", "u64", "f64"):
    for _op in ("plus", "maximum", "minimum"):
        FACTORIES["c2_segreduce_%s_%s" % (_t, _op)] = \
            (lambda t, o: lambda c: make_c2_typed(c, t, o))(_t, _op)


def traffic_table():
    """HBM bytes per launch of each workload's dominant kernel, from the table
    in profiles/hbm_traffic.md: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (KiB per
    dispatch), each scaled by what the same counter reads for a plain copy of
    known size.  A workload without a row reports null."""
    table = {}
    path = os.path.join(ROOT, "profiles", "hbm_traffic.md")
    if not os.path.exists(path):
        return table
    for line in open(path):
        cells = [c.strip() for c in line.strip().strip("|").split("|")]
        if len(cells) >= 6 and cells[0] in FACTORIES:
            try:
                fetch, ff, write, wf = (float(c.replace(",", "")) for c in cells[2:6])
            except ValueError:
                continue
            table[cells[0]] = int((fetch * ff + write * wf) * 1024)
    return table


def sustained_warmup(fn, seconds):
    """Number of warm-up steps that keep the workload running for `seconds`
    (from one timed step; at least 5)."""
    import torch
    fn(0)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(4):
        fn(i)
    torch.cuda.synchronize()
    step = (time.perf_counter() - t0) / 4
    return max(5, int(seconds / max(step, 1e-7)))


def time_steps(fn, steps, warmup):
    import torch
    for i in range(warmup):
        fn(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        fn(warmup + i)
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps


def time_each_step(fn, steps, warmup):
    """Device time of every single step: one HIP event pair per step on the
    stream the kernels run on.  Returns the sorted list in seconds."""
    import torch
    for i in range(warmup):
        fn(i)
    torch.cuda.synchronize()
    pairs = []
    for i in range(steps):
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        e0.record()
        fn(warmup + i)
        e1.record()
        pairs.append((e0, e1))
    torch.cuda.synchronize()
    return sorted(a.elapsed_time(b) / 1e3 for a, b in pairs)


def time_kernel_events(fn, steps, warmup):
    """Average duration of one launch of the dominant kernel: `steps` launches
    queued back to back between two HIP events recorded on the stream the
    kernels run on (torch's current stream), so the figure is device time per
    launch, not host launch latency."""
    import torch
    for i in range(warmup):
        fn(i)
    torch.cuda.synchronize()
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    e0.record()
    for i in range(steps):
        fn(warmup + i)
    e1.record()
    e1.synchronize()
    return e0.elapsed_time(e1) / steps / 1e3


def _time_cpu(run, budget_s):
    reps, t_total = 0, 0.0
    while reps < 1 or (t_total < budget_s and reps < 50):
        t0 = time.perf_counter()
        run()
        t_total += time.perf_counter() - t0
        reps += 1
    return t_total / reps, reps


def cpu_baseline(wk, budget_s, all_cores):
    """The CPU checker's loop timed on this host: single thread (what the
    reference's own tests run) and, for the headline workload, all the cores
    this process may use (contiguous segment ranges per thread).  Every
    repetition covers the whole workload; repetitions stop after budget_s."""
    sec1, reps1 = _time_cpu(wk.cpu(), budget_s)
    res = {"value": wk.bytes / sec1 / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
           "items_per_s": wk.items / sec1,
           "sample": "full workload, %d repetition(s), single thread, gcc -O3 -march=native "
                     "(host reports %d logical cores)" % (reps1, os.cpu_count() or 0)}
    make = getattr(wk, "cpu_threads", None)
    cores = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else 1
    cores = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores) or cores))
    if all_cores and make is not None and cores > 1:
        secn, repsn = _time_cpu(make(cores), budget_s)
        res = {"value": wk.bytes / secn / 1e9, "unit": "GB/s", "cores": cores, "kind": "port",
               "items_per_s": wk.items / secn,
               "single_thread_value": wk.bytes / sec1 / 1e9,
               "sample": "full workload, %d repetition(s) on %d threads over contiguous "
                         "segment ranges (and %d single-threaded: the single_thread_value), "
                         "gcc -O3 -march=native" % (repsn, cores, reps1)}
    return res


# Reported under 'others' in this order: first the steps on either side of the
# path (scan, reduce, lbs_segreduce, the interval moves, work creation, sorted
# search and join), then BASELINE.json's configs beside the headline one
# (configs[1]): configs[0], both halves of configs[2], configs[3], both halves
# of configs[4].  Whoever keeps only the end of the line keeps those.  About
# 55 s in all.
BASELINE_EXTRA = ("c1_segreduce_i32", "c3_load_balance_search", "c3_interval_expand_i32",
                  "c4_spmv_f32", "c5_f64max", "c5_i64sum")
DEFAULT_EXTRA = ",".join(("scan_i32", "reduce_f32", "c2_lbs_segreduce_i32",
                          "c3_interval_gather_i32", "c3_interval_scatter_i32",
                          "c3_interval_move_i32", "workcreate_i32", "sorted_search_i32",
                          "inner_join_i32") + BASELINE_EXTRA)

# The whole JSON line stays under this many characters (a record that keeps
# the last 8,000 characters of the output then holds all of it).
LINE_LIMIT = 7500

# Which yardstick (see measure_yardsticks) bounds which workload's whole call.
YARDSTICK_OF = {
    "c2_segreduce_f32": "read_nt_256MiB",
    "c3_load_balance_search": "store_1GiB_runs_read2KB",
    "c3_interval_expand_i32": "store_1GiB_runs_read4KB",
}


def sig(x, digits=5):
    """x rounded to `digits` significant digits (None and ints pass through)."""
    if x is None or isinstance(x, (int, str, bool)):
        return x
    return float("%.*g" % (digits, x))


def compact(res, yardsticks):
    """What the line keeps of a workload beside the headline."""
    r = res["roofline"]
    out = {"ms_per_step": sig(res["ms_per_step"]),
           "median_ms_per_step": sig(res["median_ms_per_step"]),
           "sustained_ms_per_step": sig(res["sustained_ms_per_step"]),
           "pct_hbm_peak": sig(res["pct_hbm_peak"], 4),
           "roofline": {"kernel": r["kernel"], "frac": sig(r["frac"], 4),
                        "kernel_ms": sig(r["kernel_ms"]), "traffic": r["traffic"]}}
    y = yardsticks.get(YARDSTICK_OF.get(res["workload"]))
    if y:
        out["frac_of_yardstick"] = sig(y / res["ms_per_step"], 4)
    if "cpu_baseline" in res:
        out["cpu_baseline"] = {"value": sig(res["cpu_baseline"]["value"], 4),
                               "cores": res["cpu_baseline"]["cores"]}
    return out


def format_line(main_res, others, yardsticks, device, steps, warmup, copies):
    """The one JSON line: the contract's keys for the headline workload, the
    yardsticks, then the other workloads (compact, BASELINE's configs last)."""
    roof = dict(main_res["roofline"])
    for k in ("achieved", "frac", "kernel_ms"):
        roof[k] = sig(roof[k])
    line = {
        "metric": "segreduce_input_GBps", "value": sig(main_res["GBps"]), "unit": "GB/s",
        "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": sig(main_res["ms_per_step"]),
        "median_ms_per_step": sig(main_res["median_ms_per_step"]),
        "sustained_ms_per_step": sig(main_res["sustained_ms_per_step"]),
        "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": main_res["dtype"],
        "data": "synthetic (seeded numpy PCG64, seed 42), inputs resident in HBM, "
                "%d rotating copies" % copies,
        "config": {"workload": main_res["workload"], "description": main_res["description"],
                   "algorithmic_bytes": main_res["algorithmic_bytes"]},
        "items_per_s": sig(main_res["items_per_s"]),
        "pct_hbm_peak": sig(main_res["pct_hbm_peak"], 4),
        "roofline": roof,
    }
    y = yardsticks.get(YARDSTICK_OF.get(main_res["workload"]))
    if y:
        line["frac_of_yardstick"] = sig(y / main_res["ms_per_step"], 4)
    if "cpu_baseline" in main_res:
        c = dict(main_res["cpu_baseline"])
        for k in ("value", "items_per_s", "single_thread_value"):
            if k in c:
                c[k] = sig(c[k], 4)
        line["cpu_baseline"] = c
    line["device"] = device
    if yardsticks:
        line["yardsticks"] = {"unit": "ms per launch; kernels that only read or only store "
                                      "(tests/csrc/test_kernels.hip), not library kernels"}
        line["yardsticks"].update({k: sig(v) for k, v in yardsticks.items()})
    if others:
        first = [k for k in others if k not in BASELINE_EXTRA]
        last = [k for k in BASELINE_EXTRA if k in others]
        line["others"] = {k: (others[k] if "error" in others[k] else
                              compact(others[k], yardsticks)) for k in first + last}
    return json.dumps(line, separators=(",", ":"))


def measure_yardsticks(steps, warmup):
    """Times of kernels that only read or only store, on this box, beside the
    library's kernels (ms per launch, `steps` launches between two
    synchronisations like a workload's steps):
      read_nt_256MiB            bare non-temporal read of 256 MiB (what the
                                2^26-float segreduce has to stream in),
                                rotating over 4 buffers
      store_1GiB_runs           1 GiB of ints stored as ragged tiles like the
                                search's, runs of 16 tiles per XCD
      store_1GiB_runs_read2KB   the same with 2 KB read per tile before it stores
                                (the search reads about that much per tile)
      store_1GiB_runs_read4KB   with 4 KB per tile (interval_expand: starts and
                                values)
      store_1GiB_eighths        the same stores, one eighth of the tiles per XCD
      read_64MiB_behind_store_1GiB   a 64 MiB read launched right behind that
                                store kernel (event pair around the read alone):
                                what a partition kernel over 2^24 starts meets
                                when it follows a call that has just stored 1 GiB"""
    import ctypes
    import torch
    tk = ctypes.CDLL(os.path.join(ROOT, "tests", "csrc", "libmgpu_test_kernels.so"))
    tk.tk_read_probe.argtypes = [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int,
                                 ctypes.c_void_p, ctypes.c_void_p]
    stream = lambda: ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    res = {}
    n = (256 << 20) // 4
    bufs = [torch.randint(0, 1 << 30, (n,), dtype=torch.int32, device="cuda")
            for _ in range(4)]

    def read(i, nbytes=256 << 20):
        rc = tk.tk_read_probe(bufs[i % 4].data_ptr(), nbytes, 1, None, stream())
        assert rc == 0, rc
    res["read_nt_256MiB"] = time_steps(read, steps, warmup) * 1e3

    probes = {"store_1GiB_runs": make_store_probe(2, 1, 0),
              "store_1GiB_runs_read2KB": make_store_probe(2, 1, 512),
              "store_1GiB_runs_read4KB": make_store_probe(2, 1, 1024),
              "store_1GiB_eighths": make_store_probe(2, 2, 0)}
    for key, wk in probes.items():
        res[key] = time_steps(wk.step, steps, warmup) * 1e3

    wk = probes["store_1GiB_runs"]
    pairs = []
    for i in range(warmup + max(steps, 10)):
        wk.step(i)
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        e0.record()
        read(i, 64 << 20)
        e1.record()
        if i >= warmup:
            pairs.append((e0, e1))
    torch.cuda.synchronize()
    res["read_64MiB_behind_store_1GiB"] = sum(a.elapsed_time(b) for a, b in pairs) / len(pairs)
    del probes, wk, bufs
    torch.cuda.empty_cache()
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=30)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="c2_segreduce_f32",
                    help="one of %s, or shape:<op>:<log2 items>:<segments> (see make_shape)"
                    % ", ".join(sorted(FACTORIES)))
    ap.add_argument("--copies", type=int, default=4)
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--no-yardsticks", action="store_true")
    ap.add_argument("--extra", default=DEFAULT_EXTRA,
                    help="comma-separated further workloads reported under 'others'")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="only run a plain 256 MiB device copy a few times: the kernel of "
                         "known traffic that rocprofv3 FETCH_SIZE/WRITE_SIZE are scaled by")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: every box of this build has one, and the "
                 "path under test uses no collective. Run with --gpus 1.")

    import torch
    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU")
    torch.cuda.set_device(0)

    if args.copy_calibration:
        n = (256 << 20) // 4
        src = torch.rand(n, dtype=torch.float32, device="cuda")
        dst = torch.empty_like(src)
        junk = torch.empty(3 * n, dtype=torch.float32, device="cuda")
        for _ in range(args.steps):
            junk.zero_()                 # push src/dst out of the 256 MB memory-side cache
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"calibration": "torch copy_", "bytes_read": n * 4,
                          "bytes_written": n * 4, "launches": args.steps}))
        return

    import moderngpu_amd as m
    import ctypes
    clock_khz, bus_bits = ctypes.c_int(0), ctypes.c_int(0)
    m.lib().mgpu_hip_memory_properties(0, ctypes.addressof(clock_khz),
                                       ctypes.addressof(bus_bits))
    traffic = traffic_table()

    def measure(key, headline):
        if key.startswith("shape:"):
            wk = make_shape(args.copies, key)
        elif key in FACTORIES:
            wk = FACTORIES[key](args.copies)
        else:
            sys.exit("unknown workload %s" % key)
        if not wk.check():
            sys.exit("parity check failed for %s: no throughput reported" % key)
        # The contract's figure: exactly `steps` steps between two
        # synchronisations, wall clock.  Beside it the median of the same
        # number of steps timed one by one with HIP events.
        sec = time_steps(wk.step, args.steps, args.warmup)
        each = time_each_step(wk.step, max(args.steps, 20), args.warmup)
        median = each[len(each) // 2]
        ksec = time_kernel_events(wk.tiles, args.steps, args.warmup)
        # Beside the burst figures above: the same K steps after 25 ms of the
        # workload running back to back (device and host at their running
        # state; long store streams then run a few per cent slower).
        sustained = time_steps(wk.step, args.steps, sustained_warmup(wk.step, 0.025))
        res = {
            "workload": key, "description": wk.name, "dtype": wk.dtype,
            "ms_per_step": sec * 1e3, "median_ms_per_step": median * 1e3,
            "sustained_ms_per_step": sustained * 1e3,
            "GBps": wk.bytes / sec / 1e9,
            "items_per_s": wk.items / sec,
            "pct_hbm_peak": 100.0 * wk.bytes / sec / 1e9 / HBM_PEAK_GBPS,
            "algorithmic_bytes": wk.bytes,
            "roofline": {
                "bound": "hbm", "kernel": wk.kernel,
                "achieved": wk.bytes / ksec / 1e9, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                "frac": wk.bytes / ksec / 1e9 / HBM_PEAK_GBPS,
                "kernel_ms": ksec * 1e3,
                "traffic": traffic.get(key),
            },
        }
        if not args.no_cpu:
            res["cpu_baseline"] = cpu_baseline(wk, 4.0 if headline else 1.5, headline)
        del wk
        torch.cuda.empty_cache()
        return res

    props = torch.cuda.get_device_properties(0)
    device = {"name": props.name, "compute_units": props.multi_processor_count,
              "hbm_peak_used_GBps": HBM_PEAK_GBPS,
              # hipDeviceProp_t's memory clock and bus width.  The reference's
              # device_prop_string prints clock x 2 x width / 8 = 4,096 GB/s
              # for the 2,000 MHz x 8,192 bits the runtime reports; HBM3E
              # moves 8 Gb/s per pin (four bits per reported clock), so the
              # fractions here are taken of the published 8 TB/s.
              "memory_clock_khz": clock_khz.value, "memory_bus_width_bits": bus_bits.value}

    main_res = measure(args.workload, True)
    others = {}
    for key in [k for k in args.extra.split(",") if k and k != args.workload]:
        # A further workload that fails (its parity check included) is
        # reported as failed; it does not take the headline with it.
        try:
            others[key] = measure(key, False)
        except (Exception, SystemExit) as e:
            others[key] = {"error": (str(e) or type(e).__name__)[:120]}
            torch.cuda.empty_cache()
    yardsticks = {}
    if not args.no_yardsticks:
        try:
            yardsticks = measure_yardsticks(args.steps, args.warmup)
        except (Exception, SystemExit) as e:
            yardsticks = {}
            print("yardsticks failed: %s" % e, file=sys.stderr)
    print(format_line(main_res, others, yardsticks, device, args.steps, args.warmup,
                      args.copies))


if __name__ == "__main__":
    main()
