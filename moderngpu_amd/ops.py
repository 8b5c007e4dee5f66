"""Host-side mirror of the mgpu:: entry points on torch device tensors.

Function names, argument meaning and error behaviour follow the reference
templates (``segreduce``, ``spmv``, ``load_balance_search``, ``transform_lbs``,
``interval_expand`` ..., see include/mgpu_hip.h for the file:line of each).
Every call goes through the C ABI of libmgpu_hip.so and is enqueued on torch's
current stream; nothing here computes on the CPU.
"""
import ctypes
import time

import torch

from ._native import lib

OPS = {"plus": 0, "maximum": 1, "minimum": 2}
_DTYPES = {torch.int32: 0, torch.int64: 2, torch.float32: 4, torch.float64: 5}
# torch has no uint32/uint64 arithmetic tensors worth using: unsigned values
# travel as the same-width signed tensors with dtype_code overridden.
_UNSIGNED = {"u32": (torch.int32, 1), "u64": (torch.int64, 3)}
_CTYPE = {0: ctypes.c_int32, 1: ctypes.c_uint32, 2: ctypes.c_int64,
          3: ctypes.c_uint64, 4: ctypes.c_float, 5: ctypes.c_double}


class MgpuError(RuntimeError):
    """A non-zero return code from libmgpu_hip (the C++ layer throws
    cuda_exception_t in the same situations)."""

    def __init__(self, code):
        self.code = code
        msg = lib().mgpu_hip_error_string(code)
        super().__init__("libmgpu_hip error %d: %s" % (
            code, msg.decode() if msg else "?"))


def _check(code):
    if code != 0:
        raise MgpuError(code)


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None and t.numel() else None


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _dev_i32(t, name):
    if t.dtype != torch.int32 or not t.is_cuda or not t.is_contiguous():
        raise TypeError("%s must be a contiguous int32 CUDA tensor" % name)
    return t


_workspaces = {}


def _workspace(nbytes, device):
    """A per-device scratch tensor that only grows.  All calls run on the
    current stream, so reuse between consecutive calls is ordered."""
    key = (device.index, torch.cuda.current_stream().cuda_stream)
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < nbytes:
        ws = torch.empty(max(int(nbytes), 1 << 16), dtype=torch.uint8, device=device)
        _workspaces[key] = ws
    return ws


_host_words = {}


def _pinned_ints(n):
    """A few ints of pinned host memory per stream, which kernels write
    straight into (the way the reference's engines take a total back: a store
    to pinned memory and a wait on the stream, no copy)."""
    key = torch.cuda.current_stream().cuda_stream
    t = _host_words.get(key)
    if t is None or t.numel() < n:
        t = torch.zeros(max(n, 8), dtype=torch.int32, pin_memory=True)
        _host_words[key] = t
    return t


def _await_words(words, n, spin_seconds=5e-3):
    """The values kernels store into words[:n] (pinned host memory, set to -1
    before the launch; the kernels store nothing negative).  A store is
    visible once its kernel has ended, which may be well before the kernels
    behind it on the stream have: the host looks at the words for a while
    before it falls back on waiting for the whole stream."""
    deadline = time.perf_counter() + spin_seconds
    while min(words[:n]) < 0:
        if time.perf_counter() > deadline:
            torch.cuda.current_stream().synchronize()
            break
    values = [int(w) for w in words[:n]]
    if min(values) < 0:
        raise MgpuError(1)
    return values


def segreduce_tile_size(dtype_code):
    return lib().mgpu_hip_segreduce_tile_size(dtype_code)


def lbs_tile_size():
    return lib().mgpu_hip_lbs_tile_size()


def lbs_search_tile_size():
    return lib().mgpu_hip_lbs_search_tile_size()


def _dtype_code(t, unsigned):
    if unsigned:
        want, code = _UNSIGNED["u32" if t.dtype == torch.int32 else "u64"]
        if t.dtype != want:
            raise TypeError("unsigned values travel as int32/int64 tensors")
        return code
    if t.dtype not in _DTYPES:
        raise TypeError("unsupported value type %s" % t.dtype)
    return _DTYPES[t.dtype]


def segreduce(values, segments, op="plus", init=0, out=None, unsigned=False,
              phases=7, workspace=None):
    """output[s] = fold of values over segment s; empty segments give init."""
    _dev_i32(segments, "segments")
    if not values.is_cuda or not values.is_contiguous():
        raise TypeError("values must be a contiguous CUDA tensor")
    code = _dtype_code(values, unsigned)
    count, nseg = values.numel(), segments.numel()
    if out is None:
        out = torch.empty(nseg, dtype=values.dtype, device=values.device)
    need = lib().mgpu_hip_segreduce_workspace_bytes(count, nseg, code)
    ws = workspace if workspace is not None else _workspace(need, values.device)
    init_c = _CTYPE[code](init)
    _check(lib().mgpu_hip_segreduce_phases(
        _ptr(values), count, _ptr(segments), nseg, _ptr(out), code, OPS[op],
        ctypes.byref(init_c), _ptr(ws), ws.numel(), _stream(), phases))
    return out


def segreduce_static(values, segments, op="plus", init=0, out=None, unsigned=False):
    """segreduce() through the entry point that allocates nothing: its
    temporaries live in a device array inside the library (4 MiB per GPU).
    Larger inputs raise MgpuError(2).  Calls on one GPU must not overlap."""
    _dev_i32(segments, "segments")
    if not values.is_cuda or not values.is_contiguous():
        raise TypeError("values must be a contiguous CUDA tensor")
    code = _dtype_code(values, unsigned)
    count, nseg = values.numel(), segments.numel()
    if out is None:
        out = torch.empty(nseg, dtype=values.dtype, device=values.device)
    init_c = _CTYPE[code](init)
    with torch.cuda.device(values.device):
        _check(lib().mgpu_hip_segreduce_static(
            _ptr(values), count, _ptr(segments), nseg, _ptr(out), code, OPS[op],
            ctypes.byref(init_c), _stream()))
    return out


def prepare_segreduce(values, segments, op="plus", init=0, out=None, unsigned=False,
                      phases=7):
    """segreduce() for a caller that repeats one call: arguments are checked
    and converted once, and the returned zero-argument callable only makes the
    C call (on the stream that is current now).  Returns (callable, out)."""
    _dev_i32(segments, "segments")
    if not values.is_cuda or not values.is_contiguous():
        raise TypeError("values must be a contiguous CUDA tensor")
    code = _dtype_code(values, unsigned)
    count, nseg = values.numel(), segments.numel()
    if out is None:
        out = torch.empty(nseg, dtype=values.dtype, device=values.device)
    need = lib().mgpu_hip_segreduce_workspace_bytes(count, nseg, code)
    ws = _workspace(need, values.device)
    init_c = _CTYPE[code](init)
    fn = lib().mgpu_hip_segreduce_phases
    args = (_ptr(values), count, _ptr(segments), nseg, _ptr(out), code, OPS[op],
            ctypes.byref(init_c), _ptr(ws), ws.numel(), _stream(), phases)
    keep = (values, segments, out, ws, init_c)      # what the pointers point at

    def call():
        _check(fn(*args))
        return keep[2]
    return call, out


def prepare_load_balance_search(count, segments, out=None, phases=3):
    """load_balance_search() prepared the same way."""
    _dev_i32(segments, "segments")
    nseg = segments.numel()
    if out is None:
        out = torch.empty(count, dtype=torch.int32, device=segments.device)
    ws = _workspace(lib().mgpu_hip_lbs_workspace_bytes(count, nseg), segments.device)
    fn = lib().mgpu_hip_load_balance_search_phases
    args = (count, _ptr(segments), nseg, _ptr(out), _ptr(ws), ws.numel(), _stream(), phases)
    keep = (segments, out, ws)

    def call():
        _check(fn(*args))
        return keep[1]
    return call, out


def transform_segreduce_mod13(count, segments, init=-1, out=None):
    """transform_segreduce with f(index) = index % 13, int32 plus."""
    _dev_i32(segments, "segments")
    nseg = segments.numel()
    if out is None:
        out = torch.empty(nseg, dtype=torch.int32, device=segments.device)
    need = lib().mgpu_hip_segreduce_workspace_bytes(count, nseg, 0)
    ws = _workspace(need, segments.device)
    _check(lib().mgpu_hip_transform_segreduce_mod13(
        count, _ptr(segments), nseg, _ptr(out), init, _ptr(ws), ws.numel(),
        _stream()))
    return out


def lbs_segreduce_seg_plus_rank(count, segments, init=-1, out=None):
    """lbs_segreduce with f(index, seg, rank) = seg + rank, int32 plus."""
    _dev_i32(segments, "segments")
    nseg = segments.numel()
    if out is None:
        out = torch.empty(nseg, dtype=torch.int32, device=segments.device)
    need = lib().mgpu_hip_segreduce_workspace_bytes(count, nseg, 0)
    ws = _workspace(need, segments.device)
    _check(lib().mgpu_hip_lbs_segreduce_seg_plus_rank(
        count, _ptr(segments), nseg, _ptr(out), init, _ptr(ws), ws.numel(),
        _stream()))
    return out


def spmv(matrix, columns, vector, segments, out=None, phases=7, workspace=None):
    """CSR y = A x; segments are the row starts (no trailing nnz entry)."""
    _dev_i32(segments, "segments")
    _dev_i32(columns, "columns")
    if matrix.dtype not in (torch.float32, torch.float64) or vector.dtype != matrix.dtype:
        raise TypeError("matrix and vector must both be float32 or float64")
    code = _DTYPES[matrix.dtype]
    count, nseg = matrix.numel(), segments.numel()
    if columns.numel() != count:
        raise ValueError("columns and matrix differ in length")
    if out is None:
        out = torch.empty(nseg, dtype=matrix.dtype, device=matrix.device)
    need = lib().mgpu_hip_segreduce_workspace_bytes(count, nseg, code)
    ws = workspace if workspace is not None else _workspace(need, matrix.device)
    _check(lib().mgpu_hip_spmv_phases(
        _ptr(matrix), _ptr(columns), _ptr(vector), count, _ptr(segments), nseg,
        _ptr(out), code, _ptr(ws), ws.numel(), _stream(), phases))
    return out


def load_balance_search(count, segments, out=None, phases=3, workspace=None):
    """out[i] = last segment whose start is <= i."""
    _dev_i32(segments, "segments")
    nseg = segments.numel()
    if out is None:
        out = torch.empty(count, dtype=torch.int32, device=segments.device)
    need = lib().mgpu_hip_lbs_workspace_bytes(count, nseg)
    ws = workspace if workspace is not None else _workspace(need, segments.device)
    _check(lib().mgpu_hip_load_balance_search_phases(
        count, _ptr(segments), nseg, _ptr(out), _ptr(ws), ws.numel(),
        _stream(), phases))
    return out


def transform_lbs(count, segments):
    """(seg, rank) per work item, the arguments transform_lbs hands its functor."""
    _dev_i32(segments, "segments")
    nseg = segments.numel()
    seg = torch.empty(count, dtype=torch.int32, device=segments.device)
    rank = torch.empty(count, dtype=torch.int32, device=segments.device)
    ws = _workspace(lib().mgpu_hip_lbs_workspace_bytes(count, nseg), segments.device)
    _check(lib().mgpu_hip_transform_lbs(
        count, _ptr(segments), nseg, _ptr(seg), _ptr(rank), _ptr(ws),
        ws.numel(), _stream()))
    return seg, rank


def _lbs_ws(count, segments):
    return _workspace(lib().mgpu_hip_lbs_workspace_bytes(count, segments.numel()),
                      segments.device)


def interval_expand(values, count, segments, out=None, phases=3, workspace=None):
    """out[i] = values[segment of i]."""
    _dev_i32(segments, "segments")
    if values.numel() != segments.numel():
        raise ValueError("one value per segment expected")
    if out is None:
        out = torch.empty(count, dtype=values.dtype, device=values.device)
    ws = workspace if workspace is not None else _lbs_ws(count, segments)
    _check(lib().mgpu_hip_interval_expand_phases(
        _ptr(values), values.element_size(), count, _ptr(segments),
        segments.numel(), _ptr(out), _ptr(ws), ws.numel(), _stream(), phases))
    return out


def interval_gather(inp, count, segments, gather, out=None):
    """out[i] = inp[gather[seg] + rank]."""
    _dev_i32(segments, "segments")
    _dev_i32(gather, "gather")
    if out is None:
        out = torch.empty(count, dtype=inp.dtype, device=inp.device)
    ws = _lbs_ws(count, segments)
    _check(lib().mgpu_hip_interval_gather(
        _ptr(inp), inp.element_size(), count, _ptr(segments), segments.numel(),
        _ptr(gather), _ptr(out), _ptr(ws), ws.numel(), _stream()))
    return out


def interval_scatter(inp, count, segments, scatter, out):
    """out[scatter[seg] + rank] = inp[i]."""
    _dev_i32(segments, "segments")
    _dev_i32(scatter, "scatter")
    ws = _lbs_ws(count, segments)
    _check(lib().mgpu_hip_interval_scatter(
        _ptr(inp), inp.element_size(), count, _ptr(segments), segments.numel(),
        _ptr(scatter), _ptr(out), _ptr(ws), ws.numel(), _stream()))
    return out


def interval_move(inp, count, segments, scatter, gather, out):
    """out[scatter[seg] + rank] = inp[gather[seg] + rank]."""
    _dev_i32(segments, "segments")
    _dev_i32(scatter, "scatter")
    _dev_i32(gather, "gather")
    ws = _lbs_ws(count, segments)
    _check(lib().mgpu_hip_interval_move(
        _ptr(inp), inp.element_size(), count, _ptr(segments), segments.numel(),
        _ptr(scatter), _ptr(gather), _ptr(out), _ptr(ws), ws.numel(), _stream()))
    return out


def load_balance_partitions(count, segments, spacing):
    """Merge-path splits every `spacing` merged elements (items + starts)."""
    _dev_i32(segments, "segments")
    n = lib().mgpu_hip_partition_count(count, segments.numel(), spacing)
    out = torch.empty(n, dtype=torch.int32, device=segments.device)
    _check(lib().mgpu_hip_load_balance_partitions(
        count, _ptr(segments), segments.numel(), spacing, _ptr(out), _stream()))
    return out


def merge_path_partitions(a_keys, a_count, b_keys, spacing, bounds="lower"):
    """Splits of the merge of two sorted int32 arrays (a_keys None = 0,1,2...)."""
    _dev_i32(b_keys, "b_keys")
    if a_keys is not None:
        _dev_i32(a_keys, "a_keys")
    n = lib().mgpu_hip_partition_count(a_count, b_keys.numel(), spacing)
    out = torch.empty(n, dtype=torch.int32, device=b_keys.device)
    _check(lib().mgpu_hip_merge_path_partitions(
        _ptr(a_keys), a_count, _ptr(b_keys), b_keys.numel(), spacing,
        1 if bounds == "upper" else 0, _ptr(out), _stream()))
    return out


def binary_search_partitions(keys, count, spacing, bounds="lower"):
    _dev_i32(keys, "keys")
    n = (count + spacing - 1) // spacing + 1
    out = torch.empty(n, dtype=torch.int32, device=keys.device)
    _check(lib().mgpu_hip_binary_search_partitions(
        _ptr(keys), count, keys.numel(), spacing,
        1 if bounds == "upper" else 0, _ptr(out), _stream()))
    return out


def scan(values, op="plus", inclusive=False, out=None, reduction=None,
         unsigned=False):
    """Device-wide scan (mgpu::scan).  Exclusive: out[0] = 0, out[i] = fold of
    values[:i]; inclusive: out[i] = fold of values[:i + 1].  The zero is only
    placed, never folded.  ``reduction`` is an optional 1-element tensor (device
    or pinned host memory) that receives the fold of everything; the returned
    pair is (out, reduction)."""
    if not values.is_cuda or not values.is_contiguous():
        raise TypeError("values must be a contiguous CUDA tensor")
    code = _dtype_code(values, unsigned)
    count = values.numel()
    if out is None:
        out = torch.empty_like(values)
    if reduction is not None and (reduction.dtype != values.dtype or reduction.numel() != 1):
        raise TypeError("reduction must be one element of the values' type")
    need = lib().mgpu_hip_scan_workspace_bytes(count, code)
    ws = _workspace(need, values.device)
    red = ctypes.c_void_p(reduction.data_ptr()) if reduction is not None else None
    _check(lib().mgpu_hip_scan(
        _ptr(values), count, _ptr(out), code, OPS[op], int(bool(inclusive)), red,
        _ptr(ws), ws.numel(), _stream()))
    return out, reduction


def reduce(values, op="plus", out=None, unsigned=False):
    """Device-wide reduction (mgpu::reduce) into a 1-element tensor; nothing
    is written for an empty input."""
    if not values.is_cuda or not values.is_contiguous():
        raise TypeError("values must be a contiguous CUDA tensor")
    code = _dtype_code(values, unsigned)
    count = values.numel()
    if out is None:
        out = torch.zeros(1, dtype=values.dtype, device=values.device)
    need = lib().mgpu_hip_reduce_workspace_bytes(count, code)
    ws = _workspace(need, values.device)
    _check(lib().mgpu_hip_reduce(
        _ptr(values), count, ctypes.c_void_p(out.data_ptr()), code, OPS[op],
        _ptr(ws), ws.numel(), _stream()))
    return out


def workcreate(created, segments):
    """Dynamic work creation (mgpu::expt::lbs_workcreate) with the per-item
    counts in a tensor: item i of the workload described by ``segments``
    creates a segment of ``created[i]`` new work-items, none if that is <= 0.

    Returns ``(new_count, new_segments, source_index, source_seg,
    source_rank)``: the number of work-items of the next pass, the start of
    each new segment, and for each new segment the item that created it, that
    item's segment and its rank there.  The sizes travel to the host between
    the two sweeps, as in the reference's engine, so this call waits for the
    stream once."""
    _dev_i32(created, "created")
    _dev_i32(segments, "segments")
    count, num_segments = created.numel(), segments.numel()
    need = lib().mgpu_hip_workcreate_workspace_bytes(count, num_segments)
    ws = _workspace(need, created.device)
    sizes = _pinned_ints(2)
    words = sizes.numpy()
    words[:2] = -1
    _check(lib().mgpu_hip_workcreate_upsweep(
        _ptr(created), count, _ptr(segments), num_segments,
        ctypes.c_void_p(sizes.data_ptr()), _ptr(ws), ws.numel(), _stream()))
    # What the second step takes besides the outputs is put together while the
    # first one runs.
    downsweep = lib().mgpu_hip_workcreate_downsweep
    front = (_ptr(created), count, _ptr(segments), num_segments)
    back = (_ptr(ws), ws.numel(), _stream())
    num_new, new_count = _await_words(words, 2)
    # One allocation for the four outputs, each row on a 256-byte boundary.
    outs = torch.empty((4, (num_new + 63) // 64 * 64), dtype=torch.int32,
                       device=created.device)[:, :num_new].unbind(0)
    if num_new:
        _check(downsweep(*front, _ptr(outs[0]), _ptr(outs[1]), _ptr(outs[2]),
                         _ptr(outs[3]), *back))
    return (new_count,) + tuple(outs)


def sorted_search(needles, haystack, bounds="lower", out=None):
    """out[i] = lower or upper bound of needles[i] in haystack
    (mgpu::sorted_search); both int32 and ascending."""
    _dev_i32(needles, "needles")
    _dev_i32(haystack, "haystack")
    n, h = needles.numel(), haystack.numel()
    if out is None:
        out = torch.empty(n, dtype=torch.int32, device=needles.device)
    ws = _workspace(lib().mgpu_hip_sorted_search_workspace_bytes(n, h), needles.device)
    _check(lib().mgpu_hip_sorted_search(
        _ptr(needles), n, _ptr(haystack), h, {"lower": 0, "upper": 1}[bounds],
        _ptr(out), _ptr(ws), ws.numel(), _stream()))
    return out


def inner_join(a, b):
    """All pairs (i, j) with a[i] == b[j] for ascending int32 keys
    (mgpu::inner_join), as an (n, 2) int32 tensor ordered by i, then j.  The
    number of pairs travels to the host between the two steps, as in the
    reference, so this call waits for the stream once."""
    _dev_i32(a, "a")
    _dev_i32(b, "b")
    na, nb = a.numel(), b.numel()
    need = lib().mgpu_hip_inner_join_workspace_bytes(na, nb)
    ws1 = torch.empty(max(int(need), 256), dtype=torch.uint8, device=a.device)
    count = _pinned_ints(1)
    word = count.numpy()
    word[:1] = -1
    _check(lib().mgpu_hip_inner_join_count(
        _ptr(a), na, _ptr(b), nb, ctypes.c_void_p(count.data_ptr()),
        _ptr(ws1), ws1.numel(), _stream()))
    n, = _await_words(word, 1)
    pairs = torch.empty((n, 2), dtype=torch.int32, device=a.device)
    if n:
        need = lib().mgpu_hip_inner_join_pairs_workspace_bytes(na, n)
        if not need:
            raise MgpuError(1)
        ws2 = _workspace(need, a.device)
        _check(lib().mgpu_hip_inner_join_pairs(
            na, nb, n, _ptr(ws1), _ptr(pairs), _ptr(ws2), ws2.numel(), _stream()))
    return pairs
