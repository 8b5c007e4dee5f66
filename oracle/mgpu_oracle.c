/*
 * TEST INFRASTRUCTURE ONLY -- CPU restatement of moderngpu's host-side loops
 * and host-callable search helpers for the merge-path / load-balancing-search /
 * segmented-reduce path.  Nothing in the product links or calls this file; it
 * is the checker that the HIP kernels are compared against, and the timed CPU
 * baseline.  Plain C99, single thread, no dependencies.
 *
 * Each function cites the reference file:line (relative to the moderngpu tree)
 * whose behaviour it restates.
 *
 * Pinning status (what independently fixes each function; see tests/):
 *   oracle_merge_path / oracle_lbs_partitions / oracle_compute_merge_range /
 *   oracle_binary_search : recorded outputs of the reference's own host-callable
 *       functions on segments={0,3,3,7}, count=10; brute-force explicit merge;
 *       split invariants.
 *   oracle_load_balance_search / oracle_transform_lbs : the reference test's
 *       vector (starts every 100, N=200030 => i/100), numpy searchsorted
 *       closed form, brute force.
 *   oracle_segreduce_* : closed form for the reference test's (index % 13)
 *       input with the reference test's generator and init=-1; numpy
 *       reduceat/fsum cross-checks; brute force.
 *   oracle_lbs_segreduce_seg_plus_rank : closed form len * seg +
 *       len * (len - 1) / 2 (mod 2^32) on the reference test's generator.
 *   oracle_cta_load_balance : per-item (segment, rank) against
 *       oracle_transform_lbs on the tile's items; every tile item written by
 *       exactly one thread; popcount of a thread's low vt merge bits = items it
 *       takes; placements consecutive (a thread ends where the next begins).
 *   oracle_workcreate : numpy flatnonzero / exclusive cumsum / searchsorted
 *       closed forms; a breadth-first search that rebuilds its frontier with
 *       it level by level (the loop of demo/bfs2.cu) against
 *       scipy.sparse.csgraph shortest path lengths.
 *   oracle_sorted_search / oracle_inner_join : numpy.searchsorted (left /
 *       right), the assertions of the reference's own test
 *       (tests/test_sortedsearch.cu:24-25), brute force over all pairs.
 *   oracle_interval_expand : numpy.repeat.
 *   oracle_spmv_* : scipy.sparse CSR product in float64.
 *   oracle_scan_* : numpy cumsum / maximum.accumulate / minimum.accumulate and
 *       the closed form of the reference's own scan test (50,000 times 1.01,
 *       tests/test_scan.cu:13-16); the reduction against numpy sum/max/min and
 *       the reference reduce test's all-ones input (tests/test_reduce.cu:14).
 */
#include <stdint.h>
#include <stddef.h>
#include <string.h>

#define ORACLE_API __attribute__((visibility("default")))

enum { OP_PLUS = 0, OP_MAXIMUM = 1, OP_MINIMUM = 2 };
enum { DT_I32 = 0, DT_U32 = 1, DT_I64 = 2, DT_U64 = 3, DT_F32 = 4, DT_F64 = 5 };

/* ------------------------------------------------------------------------- */
/* merge_path, cta_merge.hxx:8-29.  Generic over two int32 key arrays; when
 * a_keys is NULL, A is the counting sequence a_keys[i] = i (what
 * load_balance_partitions passes, search.hxx:35).  comp is less_t.
 * upper != 0 selects bounds_upper: pred = a < b, else pred = !(b < a).       */
ORACLE_API int oracle_merge_path(const int* a_keys, int a_count,
  const int* b_keys, int b_count, int diag, int upper) {
  int begin = diag - b_count; if(begin < 0) begin = 0;
  int end = diag < a_count ? diag : a_count;
  while(begin < end) {
    int mid = (int)(((int64_t)begin + end) / 2);
    int a_key = a_keys ? a_keys[mid] : mid;
    int b_key = b_keys[diag - 1 - mid];
    int pred = upper ? (a_key < b_key) : !(b_key < a_key);
    if(pred) begin = mid + 1; else end = mid;
  }
  return begin;
}

/* merge_path_partitions, search.hxx:12-27: P = div_up(a+b, spacing) + 1
 * entries, diag clamped to a_count + b_count.  Returns P.                    */
ORACLE_API int oracle_merge_path_partitions(const int* a_keys, int64_t a_count,
  const int* b_keys, int64_t b_count, int64_t spacing, int upper, int* mp) {
  int64_t total = a_count + b_count;
  int num_partitions = (int)((total + spacing - 1) / spacing) + 1;
  for(int i = 0; i < num_partitions; ++i) {
    int64_t d = spacing * i; if(d > total) d = total;
    mp[i] = oracle_merge_path(a_keys, (int)a_count, b_keys, (int)b_count,
      (int)d, upper);
  }
  return num_partitions;
}

/* load_balance_partitions, search.hxx:29-37 (counting iterator vs segment
 * starts, bounds_upper, less_t).                                             */
ORACLE_API int oracle_lbs_partitions(int64_t count, const int* segments,
  int num_segments, int spacing, int* mp) {
  return oracle_merge_path_partitions(NULL, count, segments, num_segments,
    spacing, 1, mp);
}

/* compute_merge_range, cta_merge.hxx:52-59; out = {a_begin,a_end,b_begin,b_end} */
ORACLE_API void oracle_compute_merge_range(int a_count, int b_count,
  int partition, int spacing, int mp0, int mp1, int out[4]) {
  int diag0 = spacing * partition;
  int diag1 = a_count + b_count;
  if(diag0 + spacing < diag1) diag1 = diag0 + spacing;
  out[0] = mp0; out[1] = mp1; out[2] = diag0 - mp0; out[3] = diag1 - mp1;
}

/* binary_search, cta_search.hxx:8-25 with less_t.                            */
ORACLE_API int oracle_binary_search(const int* keys, int count, int key,
  int upper) {
  int begin = 0, end = count;
  while(begin < end) {
    int mid = (int)(((int64_t)begin + end) / 2);
    int key2 = keys[mid];
    int pred = upper ? !(key < key2) : (key2 < key);
    if(pred) begin = mid + 1; else end = mid;
  }
  return begin;
}

/* binary_search_partitions, search.hxx:39-51.                                */
ORACLE_API int oracle_binary_search_partitions(const int* keys, int count,
  int num_items, int spacing, int upper, int* out) {
  int num_partitions = (count + spacing - 1) / spacing + 1;
  for(int i = 0; i < num_partitions; ++i) {
    int64_t k = (int64_t)spacing * i; if(k > count) k = count;
    out[i] = oracle_binary_search(keys, num_items, (int)k, upper);
  }
  return num_partitions;
}

/* ------------------------------------------------------------------------- */
/* Load-balancing search: seg(i) = last segment whose start <= i.  This is the
 * host statement of kernel_load_balance.hxx:78-86 with the tie rule fixed by
 * search.hxx:35-36 + cta_merge.hxx:21-23 (a segment start equal to the item
 * index is consumed before the item).  Linear merge, as in
 * tests/test_load_balance.cu:23-28's expectation lbs[i] = i / spacing.
 * Also fills rank = i - segments[seg] when rank_out != NULL
 * (cta_load_balance.hxx:165-176).                                            */
ORACLE_API void oracle_transform_lbs(int count, const int* segments,
  int num_segments, int* seg_out, int* rank_out) {
  int seg = -1;
  for(int i = 0; i < count; ++i) {
    while(seg + 1 < num_segments && segments[seg + 1] <= i) ++seg;
    if(seg_out) seg_out[i] = seg;
    if(rank_out) rank_out[i] = (seg >= 0) ? i - segments[seg] : -1;
  }
}

ORACLE_API void oracle_load_balance_search(int count, const int* segments,
  int num_segments, int* out) {
  oracle_transform_lbs(count, segments, num_segments, out, NULL);
}

/* interval_expand, kernel_intervalmove.hxx:7-20: out[i] = in[seg(i)].        */
ORACLE_API void oracle_interval_expand(const void* input, int elem_bytes,
  int count, const int* segments, int num_segments, void* output) {
  const char* in = (const char*)input; char* out = (char*)output;
  int seg = -1;
  for(int i = 0; i < count; ++i) {
    while(seg + 1 < num_segments && segments[seg + 1] <= i) ++seg;
    if(seg >= 0)
      memcpy(out + (size_t)i * elem_bytes, in + (size_t)seg * elem_bytes,
        (size_t)elem_bytes);
  }
}

/* interval_gather / interval_scatter / interval_move,
 * kernel_intervalmove.hxx:22-65 (4-byte payloads).                           */
ORACLE_API void oracle_interval_gather_i32(const int* input, int count,
  const int* segments, int num_segments, const int* gather, int* output) {
  int seg = -1;
  for(int i = 0; i < count; ++i) {
    while(seg + 1 < num_segments && segments[seg + 1] <= i) ++seg;
    if(seg >= 0) output[i] = input[gather[seg] + (i - segments[seg])];
  }
}
ORACLE_API void oracle_interval_scatter_i32(const int* input, int count,
  const int* segments, int num_segments, const int* scatter, int* output) {
  int seg = -1;
  for(int i = 0; i < count; ++i) {
    while(seg + 1 < num_segments && segments[seg + 1] <= i) ++seg;
    if(seg >= 0) output[scatter[seg] + (i - segments[seg])] = input[i];
  }
}
ORACLE_API void oracle_interval_move_i32(const int* input, int count,
  const int* segments, int num_segments, const int* scatter,
  const int* gather, int* output) {
  int seg = -1;
  for(int i = 0; i < count; ++i) {
    while(seg + 1 < num_segments && segments[seg + 1] <= i) ++seg;
    if(seg >= 0) {
      int rank = i - segments[seg];
      output[scatter[seg] + rank] = input[gather[seg] + rank];
    }
  }
}

/* ------------------------------------------------------------------------- */
/* Segmented reduce: the verification loop of tests/test_segreduce.cu:40-49:
 *   x = init; for rank in [0, size): x = rank ? op(x, y) : y;
 * i.e. init is returned for empty segments only and never folded into a
 * non-empty one.  Operators: operators.hxx:91-124 with meta.hxx:113-120's
 * max(a,b) = (a<b)?b:a and min(a,b) = (b<a)?b:a.  Integer '+' wraps.        */
#define DEF_SEGREDUCE(NAME, T, ADD)                                           \
ORACLE_API void oracle_segreduce_##NAME(const T* input, int count,           \
  const int* segments, int num_segments, T* output, int op, T init) {        \
  for(int seg = 0; seg < num_segments; ++seg) {                               \
    int begin = segments[seg];                                                \
    int end = (seg + 1 < num_segments) ? segments[seg + 1] : count;           \
    T x = init;                                                               \
    for(int k = begin; k < end; ++k) {                                        \
      T y = input[k];                                                         \
      if(k == begin) x = y;                                                   \
      else if(op == OP_PLUS) x = ADD(x, y);                                   \
      else if(op == OP_MAXIMUM) x = (x < y) ? y : x;                          \
      else x = (y < x) ? y : x;                                               \
    }                                                                         \
    output[seg] = x;                                                          \
  }                                                                           \
}
#define ADD_I32(a, b) ((int32_t)((uint32_t)(a) + (uint32_t)(b)))
#define ADD_I64(a, b) ((int64_t)((uint64_t)(a) + (uint64_t)(b)))
#define ADD_PLAIN(a, b) ((a) + (b))
DEF_SEGREDUCE(i32, int32_t, ADD_I32)
DEF_SEGREDUCE(u32, uint32_t, ADD_PLAIN)
DEF_SEGREDUCE(i64, int64_t, ADD_I64)
DEF_SEGREDUCE(u64, uint64_t, ADD_PLAIN)
DEF_SEGREDUCE(f32, float, ADD_PLAIN)
DEF_SEGREDUCE(f64, double, ADD_PLAIN)

/* Type-erased front door used by the Python wrapper. */
ORACLE_API int oracle_segreduce(const void* input, int count,
  const int* segments, int num_segments, void* output, int dtype, int op,
  const void* init) {
  switch(dtype) {
    case DT_I32: oracle_segreduce_i32((const int32_t*)input, count, segments, num_segments, (int32_t*)output, op, *(const int32_t*)init); return 0;
    case DT_U32: oracle_segreduce_u32((const uint32_t*)input, count, segments, num_segments, (uint32_t*)output, op, *(const uint32_t*)init); return 0;
    case DT_I64: oracle_segreduce_i64((const int64_t*)input, count, segments, num_segments, (int64_t*)output, op, *(const int64_t*)init); return 0;
    case DT_U64: oracle_segreduce_u64((const uint64_t*)input, count, segments, num_segments, (uint64_t*)output, op, *(const uint64_t*)init); return 0;
    case DT_F32: oracle_segreduce_f32((const float*)input, count, segments, num_segments, (float*)output, op, *(const float*)init); return 0;
    case DT_F64: oracle_segreduce_f64((const double*)input, count, segments, num_segments, (double*)output, op, *(const double*)init); return 0;
  }
  return -1;
}

/* transform_segreduce with the reference test's functor f(index) = index % 13
 * (tests/test_segreduce.cu:31-35), int32 '+'.                                */
ORACLE_API void oracle_segreduce_mod13(int count, const int* segments,
  int num_segments, int* output, int init) {
  for(int seg = 0; seg < num_segments; ++seg) {
    int begin = segments[seg];
    int end = (seg + 1 < num_segments) ? segments[seg + 1] : count;
    int x = init;
    for(int rank = 0; rank < end - begin; ++rank) {
      int y = (begin + rank) % 13;
      x = rank ? ADD_I32(x, y) : y;
    }
    output[seg] = x;
  }
}

/* lbs_segreduce, kernel_segreduce.hxx:303-404, with the functor the reference
 * test defines for it, f(index, seg, rank) = seg + rank
 * (tests/test_segreduce.cu:11-13), int32 '+': the load-balancing search hands
 * every item its segment and its rank inside the segment, the values are
 * reduced per segment, empty segments get init.                              */
ORACLE_API void oracle_lbs_segreduce_seg_plus_rank(int count,
  const int* segments, int num_segments, int* output, int init) {
  for(int seg = 0; seg < num_segments; ++seg) {
    int begin = segments[seg];
    int end = (seg + 1 < num_segments) ? segments[seg + 1] : count;
    int x = init;
    for(int rank = 0; rank < end - begin; ++rank) {
      int y = ADD_I32(seg, rank);
      x = rank ? ADD_I32(x, y) : y;
    }
    output[seg] = x;
  }
}

/* ------------------------------------------------------------------------- */
/* expt::workcreate_t, kernel_workcreate.hxx:64-247, with the per-item count
 * given as an array (the upsweep functor's return value for item `index`).
 * Upsweep (:95-122): every item with a count > 0 creates one new segment
 * (the bit test `work_count > 0`, :104) and the counts are summed.  Downsweep
 * (:169-230): the creating items, in item order, are numbered dest_seg =
 * 0, 1, ... (targets are compacted in thread order, which is item order, and
 * tiles are offset by the scan of their counts, :203-204); the start of new
 * segment dest_seg is the sum of the counts in front of it (:222-227); the
 * functor sees (dest_seg, index, seg, rank) with seg and rank from the
 * load-balancing search (:209-216).  The reference adds every count the
 * functor returns to the total, positive or not; counts <= 0 are taken as 0
 * here, which is the same for the non-negative counts it is meant for.
 * Returns the number of new segments; *new_count = number of new work-items.
 * Output arrays may be NULL (to size them first).                            */
ORACLE_API int oracle_workcreate(const int* created, int count,
  const int* segments, int num_segments, int* new_count, int* new_segments,
  int* source_index, int* source_seg, int* source_rank) {
  int dest_seg = 0, work = 0, seg = -1;
  for(int index = 0; index < count; ++index) {
    while(seg + 1 < num_segments && segments[seg + 1] <= index) ++seg;
    if(created[index] > 0) {
      if(new_segments) new_segments[dest_seg] = work;
      if(source_index) source_index[dest_seg] = index;
      if(source_seg) source_seg[dest_seg] = seg;
      if(source_rank) source_rank[dest_seg] = index - (seg >= 0 ? segments[seg] : 0);
      ++dest_seg;
      work += created[index];
    }
  }
  if(new_count) *new_count = work;
  return dest_seg;
}

/* ------------------------------------------------------------------------- */
/* sorted_search<bounds>, kernel_sortedsearch.hxx:7-73, int keys with less_t:
 * the serial merge of the two sorted arrays that the kernel performs per
 * thread (cta_merge.hxx serial_merge through merge_predicate, :41-49 here
 * restated): with bounds_lower a needle is taken while !(hay < needle), i.e.
 * in front of equal haystack keys; with bounds_upper while needle < hay fails
 * to hold for the haystack key, i.e. behind them.  indices[i] = haystack keys
 * consumed when needle i is taken (:52-57).                                  */
ORACLE_API void oracle_sorted_search(const int* needles, int num_needles,
  const int* haystack, int num_haystack, int upper, int* indices) {
  int h = 0;
  for(int i = 0; i < num_needles; ++i) {
    int key = needles[i];
    while(h < num_haystack &&
      (upper ? !(key < haystack[h]) : (haystack[h] < key))) ++h;
    indices[i] = h;
  }
}

/* inner_join, kernel_join.hxx:9-51: for every a key its matches are
 * b[lower, upper) (:14-20), the pairs are laid out by the scan of the match
 * counts (:27-31) and pair number `rank` of key `seg` is
 * (seg, lower[seg] + rank) (:41-43).  Returns the number of pairs; pairs may
 * be NULL to count only.                                                     */
ORACLE_API int64_t oracle_inner_join(const int* a, int a_count, const int* b,
  int b_count, int* pairs) {
  int64_t n = 0;
  int lo = 0, hi = 0;
  for(int i = 0; i < a_count; ++i) {
    while(lo < b_count && b[lo] < a[i]) ++lo;
    if(hi < lo) hi = lo;
    while(hi < b_count && !(a[i] < b[hi])) ++hi;
    for(int j = lo; j < hi; ++j, ++n)
      if(pairs) { pairs[2 * n] = i; pairs[2 * n + 1] = j; }
  }
  return n;
}

/* ------------------------------------------------------------------------- */
/* spmv, kernel_segreduce.hxx:285-298: y[r] = sum_k matrix[k] * x[columns[k]]
 * over the row's nonzeros in order, plus_t, init 0 (empty row => 0); row
 * starts have no trailing nnz entry.  The product is rounded to T before the
 * add, as the functor returns T (kernel_segreduce.hxx:294-295).              */
#define DEF_SPMV(NAME, T)                                                     \
ORACLE_API void oracle_spmv_##NAME(const T* matrix, const int* columns,      \
  const T* vector, int count, const int* segments, int num_segments,         \
  T* output) {                                                                \
  for(int row = 0; row < num_segments; ++row) {                               \
    int begin = segments[row];                                                \
    int end = (row + 1 < num_segments) ? segments[row + 1] : count;           \
    T x = (T)0;                                                               \
    for(int k = begin; k < end; ++k) {                                        \
      volatile T y = matrix[k] * vector[columns[k]];                          \
      x = (k == begin) ? y : x + y;                                           \
    }                                                                         \
    output[row] = x;                                                          \
  }                                                                           \
}
DEF_SPMV(f32, float)
DEF_SPMV(f64, double)

/* Row-wise sum of |a*x| in double, the normaliser of the spmv tolerance.     */
ORACLE_API void oracle_spmv_abs_f64(const void* matrix, const int* columns,
  const void* vector, int is_f64, int count, const int* segments,
  int num_segments, double* output) {
  for(int row = 0; row < num_segments; ++row) {
    int begin = segments[row];
    int end = (row + 1 < num_segments) ? segments[row + 1] : count;
    double x = 0;
    for(int k = begin; k < end; ++k) {
      double a = is_f64 ? ((const double*)matrix)[k] : ((const float*)matrix)[k];
      double v = is_f64 ? ((const double*)vector)[columns[k]] :
        ((const float*)vector)[columns[k]];
      double p = a * v; x += p < 0 ? -p : p;
    }
    output[row] = x;
  }
}

/* ------------------------------------------------------------------------- */
/* cta_load_balance_place and cta_load_balance_t::load_balance,
 * cta_load_balance.hxx:16-65 and :107-184, for tile `cta` of nv = nt * vt merged
 * elements, thread by thread.  Per thread tid: a_index[tid], b_index[tid]
 * (placement) and merge_flags[tid]; per thread and i < vt, at [tid * vt + i]:
 * the global index, segment and rank of tile item nt * i + tid (segment
 * b_begin and rank -1 past the end of the tile).  range_out = the loaded
 * range {a_begin, a_end, b_begin, b_end} of the placement.                   */
ORACLE_API void oracle_cta_load_balance(int count, const int* segments,
  int num_segments, int nt, int vt, int cta, int* a_index, int* b_index,
  int* merge_flags, int* indices, int* segs, int* ranks, int range_out[4]) {
  int nv = nt * vt;
  int total = count + num_segments;
  int diag0 = nv * cta, diag1 = diag0 + nv < total ? diag0 + nv : total;
  int mp0 = oracle_merge_path(NULL, count, segments, num_segments, diag0, 1);
  int mp1 = oracle_merge_path(NULL, count, segments, num_segments, diag1, 1);
  int a_begin = mp0, a_end = mp1, b_begin = diag0 - mp0, b_end = diag1 - mp1;
  int a_count = a_end - a_begin;

  /* cta_load_balance.hxx:21-44: starts as loaded, then `count` sentinels.    */
  int preceding = b_begin > 0;
  int lb = b_begin - preceding, le = b_end;
  if(le < num_segments && a_end < count) ++le;
  int loaded = le - lb;
  int sentinels = nv + 1 + preceding - loaded - a_count;
  int n = loaded + sentinels;
  int* b = (int*)__builtin_alloca(sizeof(int) * (size_t)(n + 2));
  for(int i = 0; i < loaded; ++i) b[i] = segments[lb + i];
  for(int i = 0; i < sentinels; ++i) b[loaded + i] = count;
  int* seg_of = (int*)__builtin_alloca(sizeof(int) * (size_t)(nv + vt + 2));

  range_out[0] = a_begin; range_out[1] = a_end;
  range_out[2] = lb; range_out[3] = le;

  for(int tid = 0; tid < nt; ++tid) {
    /* :49-63: merge path of (a_begin + i) against b with bounds_upper.       */
    int diag = vt * tid + preceding;
    int lo = diag - n > 0 ? diag - n : 0;
    int hi = diag < a_count ? diag : a_count;
    while(lo < hi) {
      int mid = (lo + hi) / 2;
      int a_key = a_begin + mid, b_key = b[diag - 1 - mid];
      if(a_key < b_key) lo = mid + 1; else hi = mid;
    }
    int mp = lo;
    a_index[tid] = a_begin + mp;
    b_index[tid] = lb + (diag - mp) - 1;

    /* :129-143: vt + 1 merge steps.                                          */
    int item = a_index[tid], segment = b_index[tid], flags = 0;
    for(int i = 0; i <= vt; ++i) {
      int p = item < b[segment + 1 - lb];
      if(p && i < vt) { seg_of[item - a_begin] = segment; ++item; }
      else ++segment;
      flags |= p << i;
    }
    merge_flags[tid] = flags;
  }
  /* :149-160: strided read-back.                                             */
  for(int tid = 0; tid < nt; ++tid)
    for(int i = 0; i < vt; ++i) {
      int j = nt * i + tid, at = tid * vt + i;
      indices[at] = a_begin + j;
      if(j < a_count) {
        segs[at] = seg_of[j];
        ranks[at] = indices[at] - b[segs[at] - lb];
      } else { segs[at] = b_begin; ranks[at] = -1; }
    }
}

/* ------------------------------------------------------------------------- */
/* Serial restatements of the CTA primitives' contracts, used to check the
 * wave64 device primitives.                                                  */

/* cta_scan_t::scan, cta_scan.hxx:42-89, and the device-wide mgpu::scan,
 * kernel_scan.hxx:11-165 (same contract with init = type_t()): exclusive or
 * inclusive scan of count values with op; init is placed at out[0] of an
 * exclusive scan and never folded; returns the reduction (init if count is
 * 0).  mgpu::reduce, kernel_reduce.hxx:11-57, is that return value.          */
#define DEF_SCAN(NAME, T, ADD)                                                \
ORACLE_API T oracle_scan_##NAME(const T* in, int count, T* out, int op,       \
  T init, int inclusive) {                                                    \
  T x = init;                                                                 \
  for(int i = 0; i < count; ++i) {                                            \
    T y = in[i];                                                              \
    T z = (i == 0) ? y : (op == OP_PLUS ? ADD(x, y) :                         \
      op == OP_MAXIMUM ? ((x < y) ? y : x) : ((y < x) ? y : x));              \
    out[i] = inclusive ? z : (i ? x : init);                                  \
    x = z;                                                                    \
  }                                                                           \
  return x;                                                                   \
}
DEF_SCAN(i32, int32_t, ADD_I32)
DEF_SCAN(u32, uint32_t, ADD_PLAIN)
DEF_SCAN(i64, int64_t, ADD_I64)
DEF_SCAN(u64, uint64_t, ADD_PLAIN)
DEF_SCAN(f32, float, ADD_PLAIN)
DEF_SCAN(f64, double, ADD_PLAIN)
