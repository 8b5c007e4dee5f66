"""ctypes binding of libmgpu_hip.so.  There is no fallback: if the library is
missing the import of any operation fails with the build command to run."""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libmgpu_hip.so")

c_int, c_i64, c_size, c_vp = ctypes.c_int, ctypes.c_int64, ctypes.c_size_t, ctypes.c_void_p

# name -> (restype, argtypes); mirrors include/mgpu_hip.h.
SIGNATURES = {
    "mgpu_hip_version": (c_int, []),
    "mgpu_hip_error_string": (ctypes.c_char_p, [c_int]),
    "mgpu_hip_memory_properties": (c_int, [c_int, c_vp, c_vp]),
    "mgpu_hip_segreduce_tile_size": (c_int, [c_int]),
    "mgpu_hip_lbs_tile_size": (c_int, []),
    "mgpu_hip_lbs_search_tile_size": (c_int, []),
    "mgpu_hip_partition_count": (c_int, [c_i64, c_i64, c_i64]),
    "mgpu_hip_load_balance_partitions": (c_int, [c_i64, c_vp, c_int, c_int, c_vp, c_vp]),
    "mgpu_hip_merge_path_partitions": (c_int, [c_vp, c_i64, c_vp, c_i64, c_i64, c_int, c_vp, c_vp]),
    "mgpu_hip_binary_search_partitions": (c_int, [c_vp, c_int, c_int, c_int, c_int, c_vp, c_vp]),
    "mgpu_hip_segreduce_workspace_bytes": (c_size, [c_int, c_int, c_int]),
    "mgpu_hip_segreduce": (c_int, [c_vp, c_int, c_vp, c_int, c_vp, c_int, c_int, c_vp, c_vp, c_size, c_vp]),
    "mgpu_hip_segreduce_static": (c_int, [c_vp, c_int, c_vp, c_int, c_vp, c_int, c_int, c_vp, c_vp]),
    "mgpu_hip_segreduce_phases": (c_int, [c_vp, c_int, c_vp, c_int, c_vp, c_int, c_int, c_vp, c_vp, c_size, c_vp, c_int]),
    "mgpu_hip_transform_segreduce_mod13": (c_int, [c_int, c_vp, c_int, c_vp, c_int, c_vp, c_size, c_vp]),
    "mgpu_hip_lbs_segreduce_seg_plus_rank": (c_int, [c_int, c_vp, c_int, c_vp, c_int, c_vp, c_size, c_vp]),
    "mgpu_hip_spmv": (c_int, [c_vp, c_vp, c_vp, c_int, c_vp, c_int, c_vp, c_int, c_vp, c_size, c_vp]),
    "mgpu_hip_spmv_phases": (c_int, [c_vp, c_vp, c_vp, c_int, c_vp, c_int, c_vp, c_int, c_vp, c_size, c_vp, c_int]),
    "mgpu_hip_lbs_workspace_bytes": (c_size, [c_int, c_int]),
    "mgpu_hip_load_balance_search": (c_int, [c_int, c_vp, c_int, c_vp, c_vp, c_size, c_vp]),
    "mgpu_hip_load_balance_search_phases": (c_int, [c_int, c_vp, c_int, c_vp, c_vp, c_size, c_vp, c_int]),
    "mgpu_hip_transform_lbs": (c_int, [c_int, c_vp, c_int, c_vp, c_vp, c_vp, c_size, c_vp]),
    "mgpu_hip_interval_expand": (c_int, [c_vp, c_int, c_int, c_vp, c_int, c_vp, c_vp, c_size, c_vp]),
    "mgpu_hip_interval_expand_phases": (c_int, [c_vp, c_int, c_int, c_vp, c_int, c_vp, c_vp, c_size, c_vp, c_int]),
    "mgpu_hip_interval_gather": (c_int, [c_vp, c_int, c_int, c_vp, c_int, c_vp, c_vp, c_vp, c_size, c_vp]),
    "mgpu_hip_interval_scatter": (c_int, [c_vp, c_int, c_int, c_vp, c_int, c_vp, c_vp, c_vp, c_size, c_vp]),
    "mgpu_hip_interval_move": (c_int, [c_vp, c_int, c_int, c_vp, c_int, c_vp, c_vp, c_vp, c_vp, c_size, c_vp]),
    "mgpu_hip_scan_workspace_bytes": (c_size, [c_int, c_int]),
    "mgpu_hip_scan": (c_int, [c_vp, c_int, c_vp, c_int, c_int, c_int, c_vp, c_vp, c_size, c_vp]),
    "mgpu_hip_reduce_workspace_bytes": (c_size, [c_int, c_int]),
    "mgpu_hip_reduce": (c_int, [c_vp, c_int, c_vp, c_int, c_int, c_vp, c_size, c_vp]),
    "mgpu_hip_sorted_search_workspace_bytes": (c_size, [c_int, c_int]),
    "mgpu_hip_sorted_search": (c_int, [c_vp, c_int, c_vp, c_int, c_int, c_vp, c_vp, c_size, c_vp]),
    "mgpu_hip_inner_join_workspace_bytes": (c_size, [c_int, c_int]),
    "mgpu_hip_inner_join_count": (c_int, [c_vp, c_int, c_vp, c_int, c_vp, c_vp, c_size, c_vp]),
    "mgpu_hip_inner_join_pairs_workspace_bytes": (c_size, [c_int, c_i64]),
    "mgpu_hip_inner_join_pairs": (c_int, [c_int, c_int, c_int, c_vp, c_vp, c_vp, c_size, c_vp]),
    "mgpu_hip_workcreate_workspace_bytes": (c_size, [c_int, c_int]),
    "mgpu_hip_workcreate_upsweep": (c_int, [c_vp, c_int, c_vp, c_int, c_vp, c_vp, c_size, c_vp]),
    "mgpu_hip_workcreate_downsweep": (c_int, [c_vp, c_int, c_vp, c_int, c_vp, c_vp, c_vp, c_vp, c_vp, c_size, c_vp]),
}

_lib = None


def library_path():
    return _SO


def lib():
    """The loaded library; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            raise ImportError(
                "libmgpu_hip.so is not built (expected at %s). Build it with "
                "`make -C moderngpu_amd/csrc` or `python -c 'import "
                "__graft_entry__ as g; g.build()'`; there is no CPU fallback."
                % _SO)
        handle = ctypes.CDLL(_SO)
        for name, (restype, argtypes) in SIGNATURES.items():
            fn = getattr(handle, name)   # AttributeError if a symbol is missing
            fn.restype = restype
            fn.argtypes = argtypes
        _lib = handle
    return _lib
