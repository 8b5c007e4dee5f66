// mgpu for AMD CDNA4: relational inner join of two sorted key arrays.
// Returns every pair (i, j) with a[i] equivalent to b[j], ordered by i, then
// j.  Interface after src/moderngpu/kernel_join.hxx:9-51.  The reference runs
// two sorted searches (lower and upper bounds of every a key in b); here one
// search finds the lower bound and the number of matches together.  Then an
// exclusive scan of the match counts, and a load-balancing search that hands every output pair its
// a index (the segment) and its position among that key's matches (the rank).
#pragma once
#include "kernel_sortedsearch.hxx"
#include "kernel_scan.hxx"
#include "kernel_load_balance.hxx"

BEGIN_MGPU_NAMESPACE

namespace detail {

// Output pair `index` of the join: (segment, first match of the segment +
// rank).  Four pairs per call go out as two 16-byte stores.
struct join_pairs_f {
  typedef void chunk_functor_tag;
  int2* output;
  MGPU_DEVICE void operator()(int index, int seg, int rank,
    tuple<int> lower) const {
    output[index] = make_int2(seg, get<0>(lower) + rank);
  }
  template<int W>
  MGPU_DEVICE void chunk(int index, const int (&seg)[W], const int (&rank)[W],
    const tuple<int> (&lower)[W]) const {
    int2 pairs[W];
    PRAGMA_UNROLL
    for(int e = 0; e < W; ++e)
      pairs[e] = make_int2(seg[e], get<0>(lower[e]) + rank[e]);
    store_consecutive<W>(output + index, pairs);
  }
};

} // namespace detail

template<typename launch_arg_t = empty_t,
  typename a_it, typename b_it, typename comp_t>
mem_t<int2> inner_join(a_it a, int a_count, b_it b, int b_count,
  comp_t comp, context_t& context) {

  {
    mem_t<int2> pairs;
    if(detail::launcher_inner_join<launch_arg_t>(a, a_count, b, b_count, comp,
      context, pairs)) return pairs;
  }

  // Matches of a[i] are b[lower[i] .. lower[i] + matches[i]): one sorted
  // search that finds both bounds of every key from the same tile of b.
  typedef typename conditional_typedef_t<launch_arg_t,
    detail::sorted_search_launch_default_t>::type_t search_launch_t;
  typedef typename std::iterator_traits<a_it>::value_type type_t;
  mem_t<int> lower(a_count, context), matches(a_count, context);
  if(a_count > 0) {
    int nv = search_launch_t::nv(context);
    mem_t<int> partitions(
      (size_t)div_up((int64_t)a_count + b_count, (int64_t)nv) + 1, context);
    mem_t<type_t> samples(
      detail::sorted_search_sample_count(a_count, b_count, nv), context);
    detail::sorted_search_launch<bounds_lower, search_launch_t>(a, a_count,
      b, b_count, lower.data(), comp, partitions.data(), samples.data(),
      context, matches.data());
  }

  // Where each key's pairs begin in the output, and how many pairs there
  // are (read back: the output has to be allocated).
  mem_t<int> starts(a_count, context);
  mem_t<int> total(1, context);
  const int* lower_data = lower.data();
  scan<scan_type_exc>(matches.data(), a_count, starts.data(), plus_t<int>(),
    total.data(), context);
  int join_count = from_mem(total)[0];

  mem_t<int2> output(join_count, context);
  transform_lbs<launch_arg_t>(detail::join_pairs_f { output.data() },
    join_count, starts.data(), a_count, mgpu::make_tuple(lower_data),
    context);
  return output;
}

END_MGPU_NAMESPACE
