"""moderngpu's load-balancing-search / segmented-reduce path on AMD MI355X.

The compute lives in ``libmgpu_hip.so`` (hand-written HIP kernels for gfx950
behind a C ABI, ``include/mgpu_hip.h``); the C++ templates with moderngpu's own
signatures are the headers under ``include/moderngpu``.  This package is the
thin Python host side used by the tests and the benchmark: torch supplies
device memory and the stream, nothing else.
"""
from .ops import (  # noqa: F401
    OPS, segreduce, transform_segreduce_mod13, spmv, load_balance_search,
    transform_lbs, interval_expand, interval_gather, interval_scatter,
    interval_move, load_balance_partitions, merge_path_partitions,
    binary_search_partitions, segreduce_tile_size, lbs_tile_size, lbs_search_tile_size, MgpuError,
    scan, reduce, lbs_segreduce_seg_plus_rank, workcreate,
    sorted_search, inner_join, prepare_segreduce, prepare_load_balance_search,
    segreduce_static,
)
from ._native import lib, library_path  # noqa: F401
