// mgpu for AMD CDNA4: scalar binary search (lower/upper bound), host and
// device (interface after src/moderngpu/cta_search.hxx:8-25), and the
// thread-serial search step over two sorted key ranges in LDS
// (src/moderngpu/cta_search.hxx:30-98).
#pragma once
#include "cta_merge.hxx"

BEGIN_MGPU_NAMESPACE

// bounds_lower: first position whose key is not less than `key`.
// bounds_upper: first position whose key is greater than `key`.
template<bounds_t bounds, typename keys_it, typename int_t, typename key_t,
  typename comp_t>
MGPU_HOST_DEVICE int_t binary_search(keys_it keys, int_t count, key_t key,
  comp_t comp) {
  int_t lo = 0, hi = count;
  while(lo < hi) {
    int_t mid = lo + (hi - lo) / 2;
    key_t probe = keys[mid];
    bool go_right = (bounds_upper == bounds) ?
      !comp(key, probe) : comp(probe, key);
    if(go_right) lo = mid + 1;
    else hi = mid;
  }
  return lo;
}

// What one thread finds walking vt steps of the merge of two sorted ranges.
template<typename type_t, int vt>
struct search_result_t {
  array_t<type_t, vt> keys;     // key taken in step i
  array_t<int, vt> indices;     // its position (plus the caller's offset)
  int decisions;                // bit i: step i took its key from A
  int matches_a;                // bit i: that A key also occurs in B
  int matches_b;                // bit i: step i took a B key that occurs in A
};

// keys_shared holds the A keys at [range.a_begin, range.a_end) and the B keys
// at [range.b_begin, range.b_end), with the B array starting at range.a_end.
// The thread merges vt keys from where its range begins -- with bounds_lower
// an A key goes in front of equal B keys, with bounds_upper behind them -- and
// notes for each whether the other array holds an equal key: an equal key of
// the other array is either the one at its head or the last one taken from it,
// depending on the tie rule, so one comparison per step decides.  Keys just in
// front of the thread's range are looked at for that (they are in the array
// whenever the index is above the array's start).  With range_check false the
// caller guarantees that neither range runs out within vt steps.
template<int vt, bounds_t bounds, bool range_check, typename type_t,
  typename comp_t>
MGPU_DEVICE search_result_t<type_t, vt>
serial_search(const type_t* keys_shared, merge_range_t range, int a_offset,
  int b_offset, comp_t comp, bool sync = true) {

  const int a_first = 0, b_first = range.a_end;
  type_t a_head = keys_shared[range.a_begin];
  type_t b_head = keys_shared[range.b_begin];
  type_t a_last = type_t(), b_last = type_t();
  if(range.a_begin > a_first) a_last = keys_shared[range.a_begin - 1];
  if(range.b_begin > b_first) b_last = keys_shared[range.b_begin - 1];

  search_result_t<type_t, vt> result = search_result_t<type_t, vt>();
  PRAGMA_UNROLL
  for(int i = 0; i < vt; ++i) {
    bool take_a = merge_predicate<bounds, range_check>(a_head, b_head, range,
      comp);
    bool a_left = !range_check || range.a_valid();
    bool b_left = !range_check || range.b_valid();
    bool a_taken = !range_check || range.a_begin > a_first;
    bool b_taken = !range_check || range.b_begin > b_first;

    bool match;
    if(take_a) {
      // lower: equal B keys are still ahead; upper: they went just before.
      match = (bounds_upper == bounds) ?
        (b_taken && !comp(b_last, a_head)) :
        (b_left && !comp(a_head, b_head));
      result.decisions |= 1 << i;
      result.matches_a |= (int)match << i;
      a_last = a_head;
    } else {
      // upper: equal A keys are still ahead; lower: they went just before.
      match = (bounds_upper == bounds) ?
        (a_left && b_left && !comp(b_head, a_head)) :
        (b_left && a_taken && !comp(a_last, b_head));
      result.matches_b |= (int)match << i;
      b_last = b_head;
    }

    int at = take_a ? range.a_begin : range.b_begin;
    result.keys[i] = take_a ? a_head : b_head;
    result.indices[i] = at + (take_a ? a_offset : b_offset);
    type_t next = keys_shared[at + 1];
    if(take_a) { a_head = next; range.a_begin = at + 1; }
    else { b_head = next; range.b_begin = at + 1; }
  }
  if(sync) __syncthreads();
  return result;
}

END_MGPU_NAMESPACE
