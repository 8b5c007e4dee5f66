"""The C-ABI library loads, exports every symbol include/mgpu_hip.h declares,
and rejects bad arguments before touching a GPU (these run without one)."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HIP_ERROR_INVALID_VALUE = 1


def _declared():
    text = open(os.path.join(ROOT, "include", "mgpu_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mgpu_hip_\w+)\s*\(", text)))


def test_header_symbols_all_exported_and_bound():
    from moderngpu_amd import _native
    names = _declared()
    assert len(names) >= 20
    handle = ctypes.CDLL(_native.library_path())
    for n in names:
        assert hasattr(handle, n), n
    assert sorted(_native.SIGNATURES) == names


def test_version_and_tile_sizes():
    import moderngpu_amd as m
    assert m.lib().mgpu_hip_version() >= 10000
    assert m.segreduce_tile_size(4) % 64 == 0 and m.segreduce_tile_size(4) > 0
    assert m.segreduce_tile_size(5) % 64 == 0 and m.segreduce_tile_size(5) > 0
    assert m.segreduce_tile_size(99) == 0
    assert m.lbs_tile_size() % 64 == 0
    assert m.lbs_search_tile_size() % 64 == 0
    assert m.lbs_search_tile_size() >= m.lbs_tile_size()     # the workspace is sized for the smaller


def test_partition_count_formula():
    import moderngpu_amd as m
    f = m.lib().mgpu_hip_partition_count
    assert f(10, 4, 7) == 3              # div_up(14, 7) + 1
    assert f(0, 0, 128) == 1
    assert f(1 << 26, 1 << 20, 4096) == ((1 << 26) + (1 << 20)) // 4096 + 1


def test_workspace_sizes():
    import moderngpu_amd as m
    L = m.lib()
    assert L.mgpu_hip_segreduce_workspace_bytes(0, 0, 4) == 0 or True
    small = L.mgpu_hip_segreduce_workspace_bytes(1000, 10, 4)
    big = L.mgpu_hip_segreduce_workspace_bytes(1 << 26, 1 << 20, 4)
    assert 0 < small < big < (1 << 22)
    assert L.mgpu_hip_segreduce_workspace_bytes(1 << 30, 1 << 30, 4) == 0  # index overflow
    assert L.mgpu_hip_segreduce_workspace_bytes(10, 10, 77) == 0           # bad dtype
    # one (items, starts) pair of ints per tile split
    assert L.mgpu_hip_lbs_workspace_bytes(1 << 28, 1 << 24) == \
        8 * (((1 << 28) + (1 << 24)) // m.lbs_tile_size() + 1 + 1)


def test_bad_arguments_are_rejected_without_a_gpu():
    import moderngpu_amd as m
    L = m.lib()
    one = ctypes.c_int(0)
    p = ctypes.byref(one)
    vp = ctypes.cast(p, ctypes.c_void_p)
    # negative sizes, bad dtype/op, null pointers, short workspace
    assert L.mgpu_hip_segreduce(vp, -1, vp, 1, vp, 0, 0, vp, vp, 1 << 20, None) == HIP_ERROR_INVALID_VALUE
    assert L.mgpu_hip_segreduce(vp, 10, vp, 1, vp, 9, 0, vp, vp, 1 << 20, None) == HIP_ERROR_INVALID_VALUE
    assert L.mgpu_hip_segreduce(vp, 10, vp, 1, vp, 0, 5, vp, vp, 1 << 20, None) == HIP_ERROR_INVALID_VALUE
    assert L.mgpu_hip_segreduce(None, 10, vp, 1, vp, 0, 0, vp, vp, 1 << 20, None) == HIP_ERROR_INVALID_VALUE
    assert L.mgpu_hip_segreduce(vp, 10, vp, 1, vp, 0, 0, vp, vp, 4, None) == HIP_ERROR_INVALID_VALUE
    assert L.mgpu_hip_segreduce(vp, 1 << 30, vp, 1 << 30, vp, 0, 0, vp, vp, 1 << 20, None) == HIP_ERROR_INVALID_VALUE
    assert L.mgpu_hip_spmv(vp, vp, vp, 10, vp, 2, vp, 0, vp, 1 << 20, None) == HIP_ERROR_INVALID_VALUE
    assert L.mgpu_hip_load_balance_search(10, None, 2, vp, vp, 1 << 20, None) == HIP_ERROR_INVALID_VALUE
    assert L.mgpu_hip_load_balance_search(10, vp, 2, vp, vp, 0, None) == HIP_ERROR_INVALID_VALUE
    assert L.mgpu_hip_interval_expand(vp, 3, 10, vp, 2, vp, vp, 1 << 20, None) == HIP_ERROR_INVALID_VALUE
    assert L.mgpu_hip_load_balance_partitions(10, vp, 2, 0, vp, None) == HIP_ERROR_INVALID_VALUE
    assert L.mgpu_hip_merge_path_partitions(None, 10, vp, 2, 8, 7, vp, None) == HIP_ERROR_INVALID_VALUE
    # workcreate: misaligned sizes, null counts, short workspace, index overflow
    buf = (ctypes.c_int * 4)()
    al = ctypes.cast(buf, ctypes.c_void_p)
    mis = ctypes.c_void_p(al.value + 4)
    assert L.mgpu_hip_workcreate_upsweep(al, 10, al, 1, mis, al, 1 << 20, None) == HIP_ERROR_INVALID_VALUE
    assert L.mgpu_hip_workcreate_upsweep(None, 10, al, 1, al, al, 1 << 20, None) == HIP_ERROR_INVALID_VALUE
    assert L.mgpu_hip_workcreate_upsweep(al, 10, al, 1, al, al, 8, None) == HIP_ERROR_INVALID_VALUE
    assert L.mgpu_hip_workcreate_downsweep(al, 10, al, 1, None, None, None, None, al, 1 << 20, None) == HIP_ERROR_INVALID_VALUE
    assert L.mgpu_hip_workcreate_workspace_bytes(1 << 30, 1 << 30) == 0
    assert 0 < L.mgpu_hip_workcreate_workspace_bytes(1000, 10) < L.mgpu_hip_workcreate_workspace_bytes(1 << 24, 1 << 20)
    assert b"invalid" in L.mgpu_hip_error_string(HIP_ERROR_INVALID_VALUE).lower()


def test_python_layer_raises_like_the_cpp_layer_throws():
    import torch
    import moderngpu_amd as m
    with pytest.raises(TypeError):
        m.segreduce(torch.zeros(4), torch.zeros(2, dtype=torch.int32))   # CPU tensors
    err = m.MgpuError(HIP_ERROR_INVALID_VALUE)
    assert err.code == HIP_ERROR_INVALID_VALUE and "invalid" in str(err).lower()
