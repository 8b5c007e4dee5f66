// mgpu for AMD CDNA4: scalar binary search (lower/upper bound), host and
// device (interface after src/moderngpu/cta_search.hxx:8-25).
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

END_MGPU_NAMESPACE
