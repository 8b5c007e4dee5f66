/*
 * libmgpu_hip -- C ABI of the MI355X (gfx950) implementation of moderngpu's
 * load-balancing-search / segmented-reduce path.
 *
 * The reference library is header-only C++ templates; it has no FFI of its
 * own.  These entry points are what its public templates bind to for raw
 * pointer arguments and the built-in operators, and what any other host
 * language binds to directly.  Each declaration cites the reference template
 * it stands for (paths relative to the moderngpu tree).
 *
 * Conventions
 *  - All pointers are device pointers unless stated otherwise.
 *  - All work is enqueued on `stream` (a hipStream_t passed as void*; NULL is
 *    the default stream).  No entry point synchronises, allocates or frees;
 *    temporaries live in the caller-provided workspace, whose required size
 *    comes from the matching *_workspace_bytes function.  The workspace must
 *    stay untouched until the enqueued work has completed.
 *  - Return value: 0 (hipSuccess) or a hipError_t code.  Nothing throws.
 *  - Index type is 32-bit int throughout, as in the reference:
 *    count + num_segments must be < 2^31.
 *  - segments[] holds the ascending start index of every segment,
 *    segments[0] == 0, with no trailing `count` entry; equal consecutive
 *    starts denote an empty segment.
 */
#ifndef MGPU_HIP_H
#define MGPU_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MGPU_HIP_API __attribute__((visibility("default")))

typedef void* mgpu_stream_t;

/* Value types (operators.hxx:91-124 are templates over the value type). */
enum {
  MGPU_I32 = 0, MGPU_U32 = 1, MGPU_I64 = 2, MGPU_U64 = 3,
  MGPU_F32 = 4, MGPU_F64 = 5
};
/* mgpu::plus_t, mgpu::maximum_t, mgpu::minimum_t (operators.hxx:91-124). */
enum { MGPU_PLUS = 0, MGPU_MAXIMUM = 1, MGPU_MINIMUM = 2 };
/* mgpu::bounds_lower / bounds_upper (types.hxx:81-84). */
enum { MGPU_BOUNDS_LOWER = 0, MGPU_BOUNDS_UPPER = 1 };
/* Phase masks for the *_phases entry points (measurement only). */
enum { MGPU_PHASE_PARTITION = 1, MGPU_PHASE_TILES = 2, MGPU_PHASE_SPINE = 4,
       MGPU_PHASE_ALL = 7,
       /* or-ed in: run the partition kernel also for calls small enough to
        * do without it (see the *_phases functions) */
       MGPU_PHASE_PARTITION_ALWAYS = 8 };

/* Library version, major * 10000 + minor * 100 + patch. */
MGPU_HIP_API int mgpu_hip_version(void);
/* Text for a return code (hipGetErrorString). */
MGPU_HIP_API const char* mgpu_hip_error_string(int code);
/* Memory clock (kHz) and bus width (bits) of `device` as hipDeviceProp_t
 * gives them -- the two numbers mgpu::device_prop_string multiplies into a
 * bandwidth figure (context.hxx:25-28): clock x 2 x width / 8. */
MGPU_HIP_API int mgpu_hip_memory_properties(int device, int* clock_khz,
  int* bus_width_bits);
/* Merged elements (items + segment starts) between consecutive tile splits:
 * what the library uses as `spacing` for segreduce on `dtype`, for the
 * load-balancing-search kernels that carry per-segment values (interval
 * expand / gather / scatter / move; the workspace is sized for this one), and
 * for those that do not (load_balance_search, transform_lbs: larger tiles). */
MGPU_HIP_API int mgpu_hip_segreduce_tile_size(int dtype);
MGPU_HIP_API int mgpu_hip_lbs_tile_size(void);
MGPU_HIP_API int mgpu_hip_lbs_search_tile_size(void);

/* ---- partitioning ------------------------------------------------------ */

/* Number of entries the partition functions write:
 * div_up(a_count + b_count, spacing) + 1  (search.hxx:18). */
MGPU_HIP_API int mgpu_hip_partition_count(int64_t a_count, int64_t b_count,
  int64_t spacing);

/* mgpu::load_balance_partitions (search.hxx:29-37): partitions[i] = merge
 * path split of cross-diagonal min(spacing * i, count + num_segments) between
 * the item indices [0, count) and the segment starts, bounds_upper. */
MGPU_HIP_API int mgpu_hip_load_balance_partitions(int64_t count,
  const int* segments, int num_segments, int spacing, int* partitions,
  mgpu_stream_t stream);

/* mgpu::merge_path_partitions<bounds> (search.hxx:12-27) for int keys with
 * less_t.  a_keys == NULL means the counting sequence 0, 1, 2, ... */
MGPU_HIP_API int mgpu_hip_merge_path_partitions(const int* a_keys,
  int64_t a_count, const int* b_keys, int64_t b_count, int64_t spacing,
  int bounds, int* partitions, mgpu_stream_t stream);

/* mgpu::binary_search_partitions<bounds> (search.hxx:39-51). */
MGPU_HIP_API int mgpu_hip_binary_search_partitions(const int* keys, int count,
  int num_items, int spacing, int bounds, int* partitions,
  mgpu_stream_t stream);

/* ---- segmented reduction ----------------------------------------------- */

/* Bytes of workspace mgpu_hip_segreduce / mgpu_hip_spmv need. */
MGPU_HIP_API size_t mgpu_hip_segreduce_workspace_bytes(int count,
  int num_segments, int dtype);

/* mgpu::segreduce (kernel_segreduce.hxx:193-268) for pointer inputs:
 * output[s] = fold of input over segment s with `op`; empty segments get
 * *init (host pointer to one value of `dtype`), which is never folded into
 * non-empty segments.  Integer sums wrap. */
MGPU_HIP_API int mgpu_hip_segreduce(const void* input, int count,
  const int* segments, int num_segments, void* output, int dtype, int op,
  const void* init, void* workspace, size_t workspace_bytes,
  mgpu_stream_t stream);

/* mgpu_hip_segreduce for callers that cannot allocate device memory (code
 * under HIP graph capture, serving loops, harnesses that forbid hipMalloc).
 * No counterpart in the reference, whose segreduce allocates its temporaries
 * through the context on every call (kernel_segreduce.hxx:210-216).  Same
 * arguments and results as mgpu_hip_segreduce without the workspace: the
 * tile splits and per-tile carries live in a device array of
 * MGPU_HIP_STATIC_SCRATCH_BYTES that the library holds on every GPU it runs
 * on until the process ends.  The call itself allocates and frees nothing.
 *  - Inputs whose workspace (mgpu_hip_segreduce_workspace_bytes) exceeds that
 *    size are rejected with hipErrorOutOfMemory (2) and nothing is enqueued;
 *    count + num_segments up to 2^28 always fits.
 *  - The device `stream` belongs to must be the current device.
 *  - All calls on one GPU share the one array: two calls may not overlap in
 *    time on the same GPU (different streams, or graphs replayed
 *    concurrently), they would race on it.  Calls on one stream are ordered
 *    and need nothing else.
 *  - The first call on each device looks the array's address up
 *    (hipGetSymbolAddress: not a stream operation, and it may load the
 *    library's code object, which allocates).  A caller that must not
 *    allocate from some point on -- one that is about to capture a graph --
 *    makes one call with count = 0 on that device before that point: it
 *    enqueues nothing and resolves the address. */
#define MGPU_HIP_STATIC_SCRATCH_BYTES (4u << 20)
MGPU_HIP_API int mgpu_hip_segreduce_static(const void* input, int count,
  const int* segments, int num_segments, void* output, int dtype, int op,
  const void* init, mgpu_stream_t stream);

/* Same, running only the selected phases (MGPU_PHASE_*).  A later phase uses
 * what an earlier complete call left in the same workspace.  For timing the
 * partition, tile and spine kernels separately.  (Inputs of up to 4,096
 * tiles have no partition kernel: their tile kernel finds its own splits,
 * unless MGPU_PHASE_PARTITION_ALWAYS is or-ed into phases.) */
MGPU_HIP_API int mgpu_hip_segreduce_phases(const void* input, int count,
  const int* segments, int num_segments, void* output, int dtype, int op,
  const void* init, void* workspace, size_t workspace_bytes,
  mgpu_stream_t stream, int phases);

/* mgpu::transform_segreduce (kernel_segreduce.hxx:272-280) with the functor
 * of the reference's own test, f(index) = index % 13, int32 plus
 * (tests/test_segreduce.cu:31-35).  Shows the generated-input path through
 * the C ABI; arbitrary functors need the C++ templates. */
MGPU_HIP_API int mgpu_hip_transform_segreduce_mod13(int count,
  const int* segments, int num_segments, int* output, int init,
  void* workspace, size_t workspace_bytes, mgpu_stream_t stream);

/* mgpu::lbs_segreduce (kernel_segreduce.hxx:303-404) with the functor of the
 * reference's own test, f(index, seg, rank) = seg + rank, int32 plus
 * (tests/test_segreduce.cu:11-13, :29-30): output[s] = sum over the items of
 * segment s of (s + rank), init for empty segments.  Shows the computed-items
 * path through the C ABI; arbitrary functors and cached iterators need the
 * C++ templates.  Workspace: mgpu_hip_segreduce_workspace_bytes(count,
 * num_segments, MGPU_I32). */
MGPU_HIP_API int mgpu_hip_lbs_segreduce_seg_plus_rank(int count,
  const int* segments, int num_segments, int* output, int init,
  void* workspace, size_t workspace_bytes, mgpu_stream_t stream);

/* mgpu::spmv (kernel_segreduce.hxx:285-298): CSR y = A * x.
 * output[r] = sum over the row's nonzeros k of matrix[k] * vector[columns[k]];
 * segments = row starts (num_segments rows, no trailing nnz entry);
 * count = number of nonzeros; dtype MGPU_F32 or MGPU_F64; empty row => 0.
 * Workspace: mgpu_hip_segreduce_workspace_bytes(count, num_segments, dtype). */
MGPU_HIP_API int mgpu_hip_spmv(const void* matrix, const int* columns,
  const void* vector, int count, const int* segments, int num_segments,
  void* output, int dtype, void* workspace, size_t workspace_bytes,
  mgpu_stream_t stream);
MGPU_HIP_API int mgpu_hip_spmv_phases(const void* matrix, const int* columns,
  const void* vector, int count, const int* segments, int num_segments,
  void* output, int dtype, void* workspace, size_t workspace_bytes,
  mgpu_stream_t stream, int phases);

/* ---- load-balancing search --------------------------------------------- */

/* Bytes of workspace the functions below need (the partition array). */
MGPU_HIP_API size_t mgpu_hip_lbs_workspace_bytes(int count, int num_segments);

/* mgpu::load_balance_search (kernel_load_balance.hxx:78-86):
 * output[i] = index of the last segment whose start is <= i, i in [0,count). */
MGPU_HIP_API int mgpu_hip_load_balance_search(int count, const int* segments,
  int num_segments, int* output, void* workspace, size_t workspace_bytes,
  mgpu_stream_t stream);
/* Same with the phases selected (MGPU_PHASE_PARTITION, MGPU_PHASE_TILES).
 * Calls of up to 1,536 tiles have no partition kernel: their tile kernel
 * finds its own splits, unless MGPU_PHASE_PARTITION_ALWAYS is or-ed in. */
MGPU_HIP_API int mgpu_hip_load_balance_search_phases(int count,
  const int* segments, int num_segments, int* output, void* workspace,
  size_t workspace_bytes, mgpu_stream_t stream, int phases);

/* mgpu::transform_lbs (kernel_load_balance.hxx:8-76) with a functor that
 * stores its arguments: seg_out[i] = segment of item i and
 * rank_out[i] = i - segments[seg_out[i]].  Either output may be NULL. */
MGPU_HIP_API int mgpu_hip_transform_lbs(int count, const int* segments,
  int num_segments, int* seg_out, int* rank_out, void* workspace,
  size_t workspace_bytes, mgpu_stream_t stream);

/* mgpu::interval_expand (kernel_intervalmove.hxx:7-20):
 * output[i] = input[segment of i] for elements of elem_bytes in
 * {1, 2, 4, 8, 16} bytes (copied bit-for-bit). */
MGPU_HIP_API int mgpu_hip_interval_expand(const void* input, int elem_bytes,
  int count, const int* segments, int num_segments, void* output,
  void* workspace, size_t workspace_bytes, mgpu_stream_t stream);
MGPU_HIP_API int mgpu_hip_interval_expand_phases(const void* input,
  int elem_bytes, int count, const int* segments, int num_segments,
  void* output, void* workspace, size_t workspace_bytes,
  mgpu_stream_t stream, int phases);

/* mgpu::interval_gather (kernel_intervalmove.hxx:22-35):
 * output[i] = input[gather[seg] + rank]. */
MGPU_HIP_API int mgpu_hip_interval_gather(const void* input, int elem_bytes,
  int count, const int* segments, int num_segments, const int* gather,
  void* output, void* workspace, size_t workspace_bytes,
  mgpu_stream_t stream);
/* mgpu::interval_scatter (kernel_intervalmove.hxx:37-50):
 * output[scatter[seg] + rank] = input[i]. */
MGPU_HIP_API int mgpu_hip_interval_scatter(const void* input, int elem_bytes,
  int count, const int* segments, int num_segments, const int* scatter,
  void* output, void* workspace, size_t workspace_bytes,
  mgpu_stream_t stream);
/* mgpu::interval_move (kernel_intervalmove.hxx:52-65):
 * output[scatter[seg] + rank] = input[gather[seg] + rank]. */
MGPU_HIP_API int mgpu_hip_interval_move(const void* input, int elem_bytes,
  int count, const int* segments, int num_segments, const int* scatter,
  const int* gather, void* output, void* workspace, size_t workspace_bytes,
  mgpu_stream_t stream);

/* ---- scan and reduce (the steps on either side of the path) ------------- */

/* Bytes of workspace mgpu_hip_scan needs for `count` items of `dtype`. */
MGPU_HIP_API size_t mgpu_hip_scan_workspace_bytes(int count, int dtype);

/* mgpu::scan / scan_event (kernel_scan.hxx:11-165) for pointer inputs.
 * inclusive == 0: output[0] = 0 and output[i] = input[0] op ... op
 * input[i - 1]; inclusive != 0: output[i] = input[0] op ... op input[i].
 * The zero is only placed, never folded (so an exclusive maximum scan of
 * negative values still starts with 0, as in the reference).  The fold of all
 * items is stored to *reduction when reduction is not NULL (device memory, or
 * host memory the device can write); for count == 0 that is 0.  input may
 * equal output. */
MGPU_HIP_API int mgpu_hip_scan(const void* input, int count, void* output,
  int dtype, int op, int inclusive, void* reduction, void* workspace,
  size_t workspace_bytes, mgpu_stream_t stream);

/* Bytes of workspace mgpu_hip_reduce needs. */
MGPU_HIP_API size_t mgpu_hip_reduce_workspace_bytes(int count, int dtype);

/* mgpu::reduce (kernel_reduce.hxx:11-57) for pointer inputs: *reduction =
 * input[0] op ... op input[count - 1]; nothing is stored for count == 0. */
MGPU_HIP_API int mgpu_hip_reduce(const void* input, int count,
  void* reduction, int dtype, int op, void* workspace,
  size_t workspace_bytes, mgpu_stream_t stream);

/* ---- dynamic work creation (the step after the search) ------------------ */

/* mgpu::expt::lbs_workcreate (kernel_workcreate.hxx:14-268) with the counts
 * read from an array: item i of a segmented workload creates a segment of
 * created[i] new work-items (none if created[i] <= 0).  Arbitrary functors
 * and cached iterators need the C++ templates.
 *
 * Bytes of workspace the two calls below share; the downsweep reads what the
 * upsweep left there. */
MGPU_HIP_API size_t mgpu_hip_workcreate_workspace_bytes(int count,
  int num_segments);

/* workcreate_t::upsweep (kernel_workcreate.hxx:64-145): stores
 * sizes[0] = number of creating items (the new num_segments) and
 * sizes[1] = sum of their counts (the new count).  sizes is 8-byte aligned
 * device memory, or host memory the device can write; it is valid once the
 * stream has reached this point. */
MGPU_HIP_API int mgpu_hip_workcreate_upsweep(const int* created, int count,
  const int* segments, int num_segments, int* sizes, void* workspace,
  size_t workspace_bytes, mgpu_stream_t stream);

/* workcreate_t::downsweep (kernel_workcreate.hxx:149-247), after an upsweep
 * with the same arguments and workspace.  For the k-th creating item (in item
 * order) stores new_segments[k] = sum of the counts of the creating items in
 * front of it, and what the reference hands its downsweep functor:
 * source_index[k] = the item, source_seg[k] = its segment, source_rank[k] =
 * its rank in that segment.  Arrays of sizes[0] ints; the source_* ones may
 * be NULL. */
MGPU_HIP_API int mgpu_hip_workcreate_downsweep(const int* created, int count,
  const int* segments, int num_segments, int* new_segments,
  int* source_index, int* source_seg, int* source_rank, void* workspace,
  size_t workspace_bytes, mgpu_stream_t stream);

/* ---- sorted search and join (callers of the search) ---------------------- */

/* Bytes of workspace mgpu_hip_sorted_search needs (the tile splits and, for
 * inputs of 2^22 keys or more, every 1,024th key of both inputs). */
MGPU_HIP_API size_t mgpu_hip_sorted_search_workspace_bytes(int num_needles,
  int num_haystack);

/* mgpu::sorted_search<bounds> (kernel_sortedsearch.hxx:7-73) for int keys
 * ordered by less_t; both arrays ascending.  indices[i] = number of haystack
 * keys less than needles[i] (MGPU_BOUNDS_LOWER) or not greater than it
 * (MGPU_BOUNDS_UPPER). */
MGPU_HIP_API int mgpu_hip_sorted_search(const int* needles, int num_needles,
  const int* haystack, int num_haystack, int bounds, int* indices,
  void* workspace, size_t workspace_bytes, mgpu_stream_t stream);

/* mgpu::inner_join (kernel_join.hxx:9-51) for ascending int keys, in the two
 * steps its data-dependent output size forces (the reference reads the count
 * back and allocates in between, :33-36).
 *
 * Step 1 (one sorted search for lower bounds and match counts where the
 * reference runs two searches, and the scan of the counts, :14-31): stores the
 * number of pairs to *join_count (device memory, or host memory the device
 * can write) and leaves what step 2 needs in `workspace`
 * (mgpu_hip_inner_join_workspace_bytes(a_count, b_count) bytes).  The count
 * (never negative) is stored by the kernel in front of the step's last one:
 * with *join_count in pinned host memory and set to -1 before the call, the
 * host may take the count as soon as the word is not negative and enqueue
 * step 2 while that last kernel still runs. */
MGPU_HIP_API size_t mgpu_hip_inner_join_workspace_bytes(int a_count,
  int b_count);
MGPU_HIP_API int mgpu_hip_inner_join_count(const int* a, int a_count,
  const int* b, int b_count, int* join_count, void* workspace,
  size_t workspace_bytes, mgpu_stream_t stream);

/* Step 2 (the load-balancing search, :38-46): pairs[2 * k] = index into a,
 * pairs[2 * k + 1] = index into b of the k-th pair, ordered by a index, then
 * b index; pairs is 8-byte aligned.  count_workspace is step 1's workspace,
 * untouched since; workspace is a second one of
 * mgpu_hip_inner_join_pairs_workspace_bytes(a_count, join_count) bytes. */
MGPU_HIP_API size_t mgpu_hip_inner_join_pairs_workspace_bytes(int a_count,
  int64_t join_count);
MGPU_HIP_API int mgpu_hip_inner_join_pairs(int a_count, int b_count,
  int join_count, const void* count_workspace, int* pairs, void* workspace,
  size_t workspace_bytes, mgpu_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* MGPU_HIP_H */
