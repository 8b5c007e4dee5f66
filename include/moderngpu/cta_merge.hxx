// mgpu for AMD CDNA4: merge-path search.  Only the pieces the
// load-balancing/segmented-reduce path needs are provided: merge_path (the
// split of one cross-diagonal), merge_predicate and compute_merge_range
// (interface after src/moderngpu/cta_merge.hxx:8-59).  The key-merging
// routines of the sorting family are not part of this library.
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

END_MGPU_NAMESPACE
