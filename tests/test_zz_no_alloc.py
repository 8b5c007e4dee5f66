"""mgpu_hip_segreduce_static, the entry point that allocates nothing (its
workspace is a device array inside the library), against mgpu_hip_segreduce
on the same inputs: two calls in a row, the second on a smaller input, so
that what the first call left in the shared array is shown not to matter."""
import ctypes

import numpy as np
import pytest
import torch

import moderngpu_amd as m
from moderngpu_amd import workloads

pytestmark = pytest.mark.gpu


def _pair(dev, values, segments, op, init):
    v = torch.from_numpy(values).to(dev)
    s = torch.from_numpy(segments).to(dev)
    want = m.segreduce(v, s, op, init)
    got = m.segreduce_static(v, s, op, init)
    torch.cuda.synchronize()
    return got.cpu().numpy(), want.cpu().numpy()


def test_static_matches_workspace_entry_point_twice(dev, oracle):
    rng = np.random.default_rng(7)
    # First call: many tiles, segments that span tiles (carries + spine).
    w = workloads.config2(scale=16)                       # 2^22 floats, 2^16 segments
    got, want = _pair(dev, w["values"], w["segments"], "plus", 0.0)
    assert np.array_equal(got, want)                      # same kernels: bit-identical
    ref = oracle.segreduce(w["values"].astype(np.float64), w["segments"], "plus", 0.0)
    assert np.all(np.abs(got - ref) <= 1e-5 * np.abs(ref) + 1e-30)

    # Second call, smaller and of another type: fewer tiles than the first
    # call left splits and carries for.
    count, nseg = 70_001, 513
    vals = rng.integers(-1000, 1000, size=count).astype(np.int64)
    segs = np.concatenate([[0], np.sort(rng.integers(0, count + 1, size=nseg - 1))]).astype(np.int32)
    got, want = _pair(dev, vals, segs, "plus", -5)
    assert np.array_equal(got, want)
    assert np.array_equal(got, oracle.segreduce(vals, segs, "plus", -5))

    # Third: a single long segment over several tiles, max.
    vals = rng.standard_normal(40_000)
    segs = np.array([0], np.int32)
    got, want = _pair(dev, vals, segs, "maximum", -np.inf)
    assert np.array_equal(got, want) and got[0] == vals.max()


def test_static_call_allocates_no_device_memory(dev):
    """After one empty call on the device (it resolves the address of the
    library's array), a call through the C ABI leaves the device's free memory
    as it was: nothing is allocated, by the library or by the runtime."""
    L = m.lib()
    w = workloads.config2(scale=64)                       # 2^20 floats, 2^14 segments
    v = torch.from_numpy(w["values"]).to(dev)
    s = torch.from_numpy(w["segments"]).to(dev)
    out = torch.empty(s.numel(), dtype=torch.float32, device=dev)
    init = ctypes.c_float(0.0)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    args = (ctypes.c_void_p(v.data_ptr()), v.numel(), ctypes.c_void_p(s.data_ptr()), s.numel(),
            ctypes.c_void_p(out.data_ptr()), 4, 0, ctypes.byref(init), stream)   # MGPU_F32, plus
    # The warm-up call: count = 0, nothing is enqueued.
    assert L.mgpu_hip_segreduce_static(None, 0, None, 0, None, 4, 0, ctypes.byref(init),
                                       stream) == 0
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info()
    for _ in range(3):
        assert L.mgpu_hip_segreduce_static(*args) == 0
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info()
    assert free_after == free_before
    want = m.segreduce(v, s, "plus", 0.0)
    assert torch.equal(out, want)


def test_static_rejects_what_does_not_fit(dev):
    L = m.lib()
    limit = 4 << 20
    # The largest 4-byte input whose workspace still fits, and one tile more.
    nv = m.segreduce_tile_size(4)
    count = 1 << 30
    assert L.mgpu_hip_segreduce_workspace_bytes(count, 0, 4) <= limit
    too_many = count
    while L.mgpu_hip_segreduce_workspace_bytes(too_many, 0, 4) <= limit:
        too_many += 64 * nv
    one = torch.zeros(4, dtype=torch.int32, device=dev)
    init = ctypes.c_int(0)
    p = ctypes.c_void_p(one.data_ptr())
    # Rejected before anything is enqueued (the pointers are never used).
    assert L.mgpu_hip_segreduce_static(p, too_many, p, 1, p, 0, 0, ctypes.byref(init), None) == 2
    assert L.mgpu_hip_segreduce_static(p, -1, p, 1, p, 0, 0, ctypes.byref(init), None) == 1
    assert L.mgpu_hip_segreduce_static(p, 10, p, 1, p, 9, 0, ctypes.byref(init), None) == 1
    # Empty input: nothing to do, no error.
    assert L.mgpu_hip_segreduce_static(None, 0, None, 0, None, 0, 0, ctypes.byref(init), None) == 0
