"""ctypes front end of ``libmgpu_oracle.so`` (the C restatement of the
reference's host loops).

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, by ``__graft_entry__.smoke``
and by ``bench.py``'s ``cpu_baseline`` leg -- never by the product package.
All arrays are numpy arrays on the host.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libmgpu_oracle.so")

OP_PLUS, OP_MAXIMUM, OP_MINIMUM = 0, 1, 2
OPS = {"plus": OP_PLUS, "maximum": OP_MAXIMUM, "minimum": OP_MINIMUM}
DTYPES = {np.dtype(np.int32): 0, np.dtype(np.uint32): 1, np.dtype(np.int64): 2,
          np.dtype(np.uint64): 3, np.dtype(np.float32): 4,
          np.dtype(np.float64): 5}


def build(force=False):
    """Compile the C restatement with the Makefile beside it."""
    if force or not os.path.exists(_SO) or \
            os.path.getmtime(_SO) < os.path.getmtime(os.path.join(_HERE, "mgpu_oracle.c")):
        subprocess.check_call(["make", "-s", "-C", _HERE, "-B", "libmgpu_oracle.so"])
    return _SO


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = ctypes.CDLL(_SO)
        _lib.oracle_scan_f32.restype = ctypes.c_float
        _lib.oracle_scan_f64.restype = ctypes.c_double
        _lib.oracle_scan_i64.restype = ctypes.c_int64
    return _lib


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p) if a is not None else None


def _i32(a):
    return np.ascontiguousarray(a, dtype=np.int32)


def merge_path(a_keys, a_count, b_keys, diag, upper=True):
    b = _i32(b_keys)
    a = None if a_keys is None else _i32(a_keys)
    return lib().oracle_merge_path(_p(a), int(a_count), _p(b), int(b.size),
                                   int(diag), int(bool(upper)))


def merge_path_partitions(a_keys, a_count, b_keys, spacing, upper=True):
    b = _i32(b_keys)
    a = None if a_keys is None else _i32(a_keys)
    n = (int(a_count) + b.size + spacing - 1) // spacing + 1
    mp = np.empty(n, dtype=np.int32)
    got = lib().oracle_merge_path_partitions(
        _p(a), ctypes.c_int64(int(a_count)), _p(b), ctypes.c_int64(b.size),
        ctypes.c_int64(int(spacing)), int(bool(upper)), _p(mp))
    assert got == n
    return mp


def lbs_partitions(count, segments, spacing):
    return merge_path_partitions(None, count, segments, spacing, True)


def compute_merge_range(a_count, b_count, partition, spacing, mp0, mp1):
    out = np.empty(4, dtype=np.int32)
    lib().oracle_compute_merge_range(int(a_count), int(b_count), int(partition),
                                     int(spacing), int(mp0), int(mp1), _p(out))
    return tuple(int(x) for x in out)


def binary_search(keys, key, upper=False):
    k = _i32(keys)
    return lib().oracle_binary_search(_p(k), int(k.size), int(key), int(bool(upper)))


def binary_search_partitions(keys, count, spacing, upper=False):
    k = _i32(keys)
    n = (int(count) + spacing - 1) // spacing + 1
    out = np.empty(n, dtype=np.int32)
    lib().oracle_binary_search_partitions(_p(k), int(count), int(k.size),
                                          int(spacing), int(bool(upper)), _p(out))
    return out


def transform_lbs(count, segments):
    s = _i32(segments)
    seg = np.empty(count, dtype=np.int32)
    rank = np.empty(count, dtype=np.int32)
    lib().oracle_transform_lbs(int(count), _p(s), int(s.size), _p(seg), _p(rank))
    return seg, rank


def load_balance_search(count, segments):
    s = _i32(segments)
    out = np.empty(count, dtype=np.int32)
    lib().oracle_load_balance_search(int(count), _p(s), int(s.size), _p(out))
    return out


def interval_expand(values, count, segments):
    s = _i32(segments)
    v = np.ascontiguousarray(values)
    out = np.zeros(count, dtype=v.dtype)
    lib().oracle_interval_expand(_p(v), int(v.dtype.itemsize), int(count), _p(s),
                                 int(s.size), _p(out))
    return out


def interval_gather(inp, count, segments, gather):
    s, g, x = _i32(segments), _i32(gather), _i32(inp)
    out = np.zeros(count, dtype=np.int32)
    lib().oracle_interval_gather_i32(_p(x), int(count), _p(s), int(s.size), _p(g), _p(out))
    return out


def interval_scatter(inp, count, segments, scatter, out_size):
    s, g, x = _i32(segments), _i32(scatter), _i32(inp)
    out = np.zeros(out_size, dtype=np.int32)
    lib().oracle_interval_scatter_i32(_p(x), int(count), _p(s), int(s.size), _p(g), _p(out))
    return out


def interval_move(inp, count, segments, scatter, gather, out_size):
    s, sc, g, x = _i32(segments), _i32(scatter), _i32(gather), _i32(inp)
    out = np.zeros(out_size, dtype=np.int32)
    lib().oracle_interval_move_i32(_p(x), int(count), _p(s), int(s.size), _p(sc), _p(g), _p(out))
    return out


def segreduce(values, segments, op="plus", init=0):
    v = np.ascontiguousarray(values)
    s = _i32(segments)
    out = np.empty(s.size, dtype=v.dtype)
    ini = np.array([init], dtype=v.dtype)
    rc = lib().oracle_segreduce(_p(v), int(v.size), _p(s), int(s.size), _p(out),
                                DTYPES[v.dtype], OPS[op], _p(ini))
    assert rc == 0
    return out


def segreduce_threads(values, segments, op="plus", init=0, threads=1):
    """The same loop run by `threads` host threads, each over a contiguous
    range of segments holding about the same number of items (the C call
    releases the GIL).  Used as the all-cores CPU baseline."""
    from concurrent.futures import ThreadPoolExecutor
    v = np.ascontiguousarray(values)
    s = _i32(segments)
    out = np.empty(s.size, dtype=v.dtype)
    ini = np.array([init], dtype=v.dtype)
    if threads <= 1 or s.size < 2 * threads:
        return segreduce(values, segments, op, init)
    # segment index where each thread starts: balanced by items
    cuts = np.searchsorted(s, np.arange(1, threads) * (v.size // threads), side="left")
    bounds = [0] + [int(c) for c in cuts] + [int(s.size)]
    fn = lib().oracle_segreduce
    dt, opc = DTYPES[v.dtype], OPS[op]
    sp, op_, vp, ip = s.ctypes.data, out.ctypes.data, _p(v), _p(ini)

    def run(k):
        b, e = bounds[k], bounds[k + 1]
        if e <= b:
            return 0
        end_item = int(s[e]) if e < s.size else int(v.size)
        return fn(vp, end_item, ctypes.c_void_p(sp + 4 * b), e - b,
                  ctypes.c_void_p(op_ + v.itemsize * b), dt, opc, ip)

    with ThreadPoolExecutor(max_workers=threads) as pool:
        assert all(rc == 0 for rc in pool.map(run, range(threads)))
    return out


def segreduce_mod13(count, segments, init=-1):
    s = _i32(segments)
    out = np.empty(s.size, dtype=np.int32)
    lib().oracle_segreduce_mod13(int(count), _p(s), int(s.size), _p(out), int(init))
    return out


def lbs_segreduce_seg_plus_rank(count, segments, init=-1):
    s = _i32(segments)
    out = np.empty(s.size, dtype=np.int32)
    lib().oracle_lbs_segreduce_seg_plus_rank(int(count), _p(s), int(s.size), _p(out),
                                             int(init))
    return out


def workcreate(created, segments):
    """(new_count, new_segments, source_index, source_seg, source_rank) of
    expt::lbs_workcreate with the per-item counts in ``created``."""
    c, s = _i32(created), _i32(segments)
    fn = lib().oracle_workcreate
    fn.restype = ctypes.c_int
    new_count = ctypes.c_int(0)
    n = fn(_p(c), int(c.size), _p(s), int(s.size), ctypes.byref(new_count),
           None, None, None, None)
    outs = [np.empty(n, dtype=np.int32) for _ in range(4)]
    fn(_p(c), int(c.size), _p(s), int(s.size), ctypes.byref(new_count),
       _p(outs[0]), _p(outs[1]), _p(outs[2]), _p(outs[3]))
    return (new_count.value,) + tuple(outs)


def sorted_search(needles, haystack, upper=False):
    n, h = _i32(needles), _i32(haystack)
    out = np.empty(n.size, dtype=np.int32)
    lib().oracle_sorted_search(_p(n), int(n.size), _p(h), int(h.size), int(bool(upper)),
                               _p(out))
    return out


def inner_join(a, b):
    """(n, 2) int32 array of (a index, b index), ordered by a index then b."""
    x, y = _i32(a), _i32(b)
    fn = lib().oracle_inner_join
    fn.restype = ctypes.c_int64
    n = fn(_p(x), int(x.size), _p(y), int(y.size), None)
    pairs = np.empty((n, 2), dtype=np.int32)
    fn(_p(x), int(x.size), _p(y), int(y.size), _p(pairs))
    return pairs


def cta_load_balance(count, segments, nt, vt, cta):
    """One tile of cta_load_balance_t::load_balance, thread by thread."""
    s = _i32(segments)
    a_index = np.empty(nt, dtype=np.int32)
    b_index = np.empty(nt, dtype=np.int32)
    flags = np.empty(nt, dtype=np.int32)
    indices = np.empty(nt * vt, dtype=np.int32)
    segs = np.empty(nt * vt, dtype=np.int32)
    ranks = np.empty(nt * vt, dtype=np.int32)
    rng = np.empty(4, dtype=np.int32)
    lib().oracle_cta_load_balance(int(count), _p(s), int(s.size), int(nt), int(vt),
                                  int(cta), _p(a_index), _p(b_index), _p(flags),
                                  _p(indices), _p(segs), _p(ranks), _p(rng))
    return {"a_index": a_index, "b_index": b_index, "merge_flags": flags,
            "indices": indices.reshape(nt, vt), "segments": segs.reshape(nt, vt),
            "ranks": ranks.reshape(nt, vt), "range": rng}


def spmv(matrix, columns, vector, segments):
    m = np.ascontiguousarray(matrix)
    x = np.ascontiguousarray(vector, dtype=m.dtype)
    c, s = _i32(columns), _i32(segments)
    out = np.empty(s.size, dtype=m.dtype)
    fn = lib().oracle_spmv_f32 if m.dtype == np.float32 else lib().oracle_spmv_f64
    fn(_p(m), _p(c), _p(x), int(m.size), _p(s), int(s.size), _p(out))
    return out


def spmv_abs(matrix, columns, vector, segments):
    m = np.ascontiguousarray(matrix)
    x = np.ascontiguousarray(vector, dtype=m.dtype)
    c, s = _i32(columns), _i32(segments)
    out = np.empty(s.size, dtype=np.float64)
    lib().oracle_spmv_abs_f64(_p(m), _p(c), _p(x), int(m.dtype == np.float64),
                              int(m.size), _p(s), int(s.size), _p(out))
    return out


def scan(values, op="plus", init=0, inclusive=False):
    v = np.ascontiguousarray(values)
    out = np.empty_like(v)
    name = {np.dtype(np.int32): "i32", np.dtype(np.int64): "i64",
            np.dtype(np.uint32): "u32", np.dtype(np.uint64): "u64",
            np.dtype(np.float32): "f32", np.dtype(np.float64): "f64"}[v.dtype]
    fn = getattr(lib(), "oracle_scan_" + name)
    ct = {"i32": ctypes.c_int32, "i64": ctypes.c_int64, "u32": ctypes.c_uint32,
          "u64": ctypes.c_uint64, "f32": ctypes.c_float,
          "f64": ctypes.c_double}[name]
    fn.restype = ct
    fn.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p, ctypes.c_int,
                   ct, ctypes.c_int]
    red = fn(_p(v), int(v.size), _p(out), OPS[op], ct(init), int(bool(inclusive)))
    return out, red
