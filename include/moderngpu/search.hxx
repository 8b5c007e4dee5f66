// mgpu for AMD CDNA4: partition kernels.  One search per tile boundary cuts a
// merge (or a load-balancing search) into tiles of `spacing` merged elements;
// the tile kernels then run independently.  Interface after
// src/moderngpu/search.hxx:12-51.
#pragma once

#include "loadstore.hxx"
#include "operators.hxx"
#include "cta_search.hxx"
#include "memory.hxx"
#include "context.hxx"

BEGIN_MGPU_NAMESPACE

namespace detail {

// Kernel body shared by the template entry point and the C launcher:
// p[index] = merge-path split of cross-diagonal min(spacing * index, total).
template<bounds_t bounds, typename int_t, typename a_keys_it,
  typename b_keys_it, typename comp_t>
struct merge_path_partition_f {
  a_keys_it a; b_keys_it b;
  int64_t a_count, b_count, spacing;
  comp_t comp;
  int_t* p;

  MGPU_DEVICE void operator()(int index) const {
    int64_t total = a_count + b_count;
    int64_t d = spacing * index;
    int_t diag = (int_t)(d < total ? d : total);
    p[index] = merge_path<bounds>(a, (int_t)a_count, b, (int_t)b_count,
      diag, comp);
  }
};

} // namespace detail

// Writes div_up(a_count + b_count, spacing) + 1 splits into p (device
// memory) on the context's stream.  Returns the number of splits.
template<bounds_t bounds, typename a_keys_it, typename b_keys_it,
  typename comp_t, typename int_t>
int merge_path_partitions_into(a_keys_it a, int64_t a_count, b_keys_it b,
  int64_t b_count, int64_t spacing, comp_t comp, int_t* p,
  context_t& context) {
  int num_partitions = (int)div_up(a_count + b_count, spacing) + 1;
  detail::merge_path_partition_f<bounds, int_t, a_keys_it, b_keys_it, comp_t>
    f { a, b, a_count, b_count, spacing, comp, p };
  transform<256>(f, num_partitions, context);
  return num_partitions;
}

template<bounds_t bounds, typename a_keys_it, typename b_keys_it,
  typename comp_t>
mem_t<typename std::iterator_traits<a_keys_it>::value_type>
merge_path_partitions(a_keys_it a, int64_t a_count, b_keys_it b,
  int64_t b_count, int64_t spacing, comp_t comp, context_t& context) {

  typedef typename std::iterator_traits<a_keys_it>::value_type int_t;
  int num_partitions = (int)div_up(a_count + b_count, spacing) + 1;
  mem_t<int_t> mem(num_partitions, context);
  merge_path_partitions_into<bounds>(a, a_count, b, b_count, spacing, comp,
    mem.data(), context);
  return mem;
}

// Splits of the merge of work-item indices [0, dest_count) with the segment
// starts: tile i owns items [mp[i], mp[i + 1]) and the segments whose start
// falls between the two cross-diagonals.
template<typename segments_it>
auto load_balance_partitions(int64_t dest_count, segments_it segments,
  int num_segments, int spacing, context_t& context) ->
  mem_t<typename std::iterator_traits<segments_it>::value_type> {

  typedef typename std::iterator_traits<segments_it>::value_type int_t;
  return merge_path_partitions<bounds_upper>(counting_iterator_t<int_t>(0),
    dest_count, segments, num_segments, spacing, less_t<int_t>(), context);
}

// p[i] = lower/upper bound of min(spacing * i, count) in keys[0, num_items).
template<bounds_t bounds, typename keys_it>
mem_t<int> binary_search_partitions(keys_it keys, int count, int num_items,
  int spacing, context_t& context) {

  int num_partitions = div_up(count, spacing) + 1;
  mem_t<int> mem(num_partitions, context);
  int* p = mem.data();
  transform<256>([=]MGPU_DEVICE(int index) {
    int key = (int)min((int64_t)spacing * index, (int64_t)count);
    p[index] = binary_search<bounds>(keys, num_items, key, less_t<int>());
  }, num_partitions, context);
  return mem;
}

END_MGPU_NAMESPACE
