// mgpu for AMD CDNA4: merge-path search -- merge_path (the split of one
// cross-diagonal), merge_predicate and compute_merge_range (interface after
// src/moderngpu/cta_merge.hxx:8-59), which is what the load-balancing search
// and the segmented reduction stand on -- and the CTA-level merge of two key
// ranges (:63-212): both ranges into LDS as one array, a merge-path search per
// thread, vt merged keys per thread.  The library's own kernels use the first
// part only; the second is here for callers who built merge-style kernels
// from it.
#pragma once
#include "loadstore.hxx"

BEGIN_MGPU_NAMESPACE

// Cross-diagonal `diag` of the merge of A (a_count keys) and B (b_count
// keys): returns how many of the first diag merged keys come from A.
//   bounds_lower: equal keys are taken from A first (stable merge).
//   bounds_upper: equal keys are taken from B first.  With A = work-item
//     indices and B = segment starts this puts a segment's start in front of
//     the first item of the segment, which is the load-balancing-search rule
//     "an item belongs to the last segment that starts at or before it".
// The midpoint is computed without overflow for counts up to 2^31 - 1.
template<bounds_t bounds = bounds_lower, typename a_keys_it,
  typename b_keys_it, typename int_t, typename comp_t>
MGPU_HOST_DEVICE int_t merge_path(a_keys_it a_keys, int_t a_count,
  b_keys_it b_keys, int_t b_count, int_t diag, comp_t comp) {

  typedef typename std::iterator_traits<a_keys_it>::value_type type_t;
  int_t lo = (diag > b_count) ? (int_t)(diag - b_count) : (int_t)0;
  int_t hi = (diag < a_count) ? diag : a_count;

  while(lo < hi) {
    int_t mid = lo + (hi - lo) / 2;
    type_t a_key = a_keys[mid];
    type_t b_key = b_keys[diag - 1 - mid];
    bool take_a = (bounds_upper == bounds) ?
      comp(a_key, b_key) : !comp(b_key, a_key);
    if(take_a) lo = mid + 1;
    else hi = mid;
  }
  return lo;
}

// Both inputs live in one array; range gives their positions.
template<bounds_t bounds, typename keys_it, typename comp_t>
MGPU_HOST_DEVICE int merge_path(keys_it keys, merge_range_t range,
  int diag, comp_t comp) {
  return merge_path<bounds>(
    keys + range.a_begin, range.a_count(),
    keys + range.b_begin, range.b_count(), diag, comp);
}

template<bounds_t bounds, bool range_check, typename type_t, typename comp_t>
MGPU_HOST_DEVICE bool merge_predicate(type_t a_key, type_t b_key,
  merge_range_t range, comp_t comp) {
  if(range_check && range.a_begin >= range.a_end) return false;
  if(range_check && range.b_begin >= range.b_end) return true;
  return (bounds_upper == bounds) ? comp(a_key, b_key) : !comp(b_key, a_key);
}

// Tile `partition` of a merge cut every `spacing` merged elements, given the
// merge-path splits at its two ends: items [mp0, mp1) of A and the matching
// part of B.
MGPU_HOST_DEVICE merge_range_t compute_merge_range(int a_count, int b_count,
  int partition, int spacing, int mp0, int mp1) {
  int diag0 = spacing * partition;
  int diag1 = diag0 + min(spacing, a_count + b_count - diag0);
  return merge_range_t { mp0, mp1, diag0 - mp0, diag1 - mp1 };
}

////////////////////////////////////////////////////////////////////////////////
// Two ranges addressed as one: element j is a[j] for j < a_count and
// b[j - a_count] behind that.

namespace detail {
template<typename type_t, typename a_it, typename b_it>
MGPU_DEVICE type_t two_streams_at(a_it a, int a_count, b_it b, int j) {
  if(j < a_count) return a[j];
  return b[j - a_count];
}
} // namespace detail

// Strided order: x[i] = element nt * i + tid, for elements that exist.
template<int nt, int vt, typename type_t, typename a_it, typename b_it>
MGPU_DEVICE array_t<type_t, vt> load_two_streams_reg(a_it a, int a_count,
  b_it b, int b_count, int tid) {
  array_t<type_t, vt> x;
  int total = a_count + b_count;
  PRAGMA_UNROLL
  for(int i = 0; i < vt; ++i) {
    int j = nt * i + tid;
    if(j < total) x[i] = detail::two_streams_at<type_t>(a, a_count, b, j);
  }
  return x;
}

// The same into LDS: shared[j] = element j.  Slots from the total up to
// nt * vt are written too (with whatever the registers hold), as the strided
// register store does not look at the count.
template<int nt, int vt, typename a_it, typename b_it, typename type_t,
  int shared_size>
MGPU_DEVICE void load_two_streams_shared(a_it a, int a_count, b_it b,
  int b_count, int tid, type_t (&shared)[shared_size], bool sync = true) {
  array_t<type_t, vt> x = load_two_streams_reg<nt, vt, type_t>(a, a_count, b,
    b_count, tid);
  reg_to_shared_strided<nt>(x, tid, shared, sync);
}

// x[i] = element indices[i] of the two ranges, for the slots nt * i + tid
// that lie below a_count + b_count; and the same stored to c in strided order.
template<int nt, int vt, typename type_t, typename a_it, typename b_it>
MGPU_DEVICE array_t<type_t, vt> gather_two_streams_strided(a_it a,
  int a_count, b_it b, int b_count, array_t<int, vt> indices, int tid) {
  array_t<type_t, vt> x;
  int total = a_count + b_count;
  PRAGMA_UNROLL
  for(int i = 0; i < vt; ++i)
    if(nt * i + tid < total)
      x[i] = detail::two_streams_at<type_t>(a, a_count, b, indices[i]);
  return x;
}
template<int nt, int vt, typename a_it, typename b_it, typename c_it>
MGPU_DEVICE void transfer_two_streams_strided(a_it a, int a_count, b_it b,
  int b_count, array_t<int, vt> indices, int tid, c_it c) {
  typedef typename std::iterator_traits<a_it>::value_type type_t;
  array_t<type_t, vt> x = gather_two_streams_strided<nt, vt, type_t>(a,
    a_count, b, b_count, indices, tid);
  reg_to_mem_strided<nt>(x, tid, a_count + b_count, c);
}

////////////////////////////////////////////////////////////////////////////////
// One thread merges vt keys, starting where its range begins.  keys_shared
// holds both arrays; keys[i] is the i-th merged key and indices[i] where it
// sits in keys_shared (past the end of both ranges: copies of the last state,
// meaningless).

template<bounds_t bounds, int vt, typename type_t, typename comp_t>
MGPU_DEVICE merge_pair_t<type_t, vt> serial_merge(const type_t* keys_shared,
  merge_range_t range, comp_t comp, bool sync = true) {
  // The head of a range that has run out is never compared, so it is not
  // read either: every read stays inside the two ranges.
  type_t a_head = type_t(), b_head = type_t();
  if(range.a_valid()) a_head = keys_shared[range.a_begin];
  if(range.b_valid()) b_head = keys_shared[range.b_begin];
  merge_pair_t<type_t, vt> merged;
  PRAGMA_UNROLL
  for(int i = 0; i < vt; ++i) {
    bool take_a = merge_predicate<bounds, true>(a_head, b_head, range, comp);
    int at = take_a ? range.a_begin : range.b_begin;
    merged.keys[i] = take_a ? a_head : b_head;
    merged.indices[i] = at;
    if(take_a) {
      ++range.a_begin;
      if(range.a_valid()) a_head = keys_shared[range.a_begin];
    } else {
      ++range.b_begin;
      if(range.b_valid()) b_head = keys_shared[range.b_begin];
    }
  }
  if(sync) __syncthreads();
  return merged;
}

// A tile of the merge of a and b: range_mem gives the tile's parts of the two
// arrays; they are staged in keys_shared (A, then B), every thread finds its
// cross-diagonal vt * tid and merges vt keys.  indices[] are positions in
// keys_shared.
template<bounds_t bounds, int nt, int vt, typename a_it, typename b_it,
  typename type_t, typename comp_t, int shared_size>
MGPU_DEVICE merge_pair_t<type_t, vt> cta_merge_from_mem(a_it a, b_it b,
  merge_range_t range_mem, int tid, comp_t comp,
  type_t (&keys_shared)[shared_size]) {
  static_assert(shared_size >= nt * vt + 1,
    "cta_merge_from_mem needs nt * vt + 1 elements of LDS");
  load_two_streams_shared<nt, vt>(a + range_mem.a_begin, range_mem.a_count(),
    b + range_mem.b_begin, range_mem.b_count(), tid, keys_shared, true);
  merge_range_t local = range_mem.to_local();
  int diag = min(vt * tid, local.total());
  int mp = merge_path<bounds>(keys_shared, local, diag, comp);
  return serial_merge<bounds, vt>(keys_shared, local.partition(mp, diag),
    comp);
}

END_MGPU_NAMESPACE
