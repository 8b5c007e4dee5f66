// mgpu for AMD CDNA4: relational inner join of two sorted key arrays.
// Returns every pair (i, j) with a[i] equivalent to b[j], ordered by i, then
// j.  Interface after src/moderngpu/kernel_join.hxx:9-51.  The reference runs
// two sorted searches (lower and upper bounds of every a key in b); here one
// search finds the lower bound and the number of matches together, and adds
// the matches up by tiles of the scan that follows, which so starts from its
// partials and reads the match counts once.  Then that exclusive scan, and a
// load-balancing search that hands every output pair its a index (the
// segment) and its position among that key's matches (the rank).
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

// The join's first step with its temporaries in caller-provided device
// memory: lower[i] = first b key equivalent to a[i], matches[i] = how many
// are, starts = exclusive scan of matches, *join_count = number of pairs.
// partitions and samples as for sorted_search_launch; partials holds
// scan_partials_count(a_count, nv of the scan) ints.  The event, when not
// null, is recorded as soon as *join_count has been written, which is before
// the last kernel of the scan.
template<typename search_launch_t, typename a_it, typename b_it,
  typename comp_t, typename reduction_it>
void join_count_launch(a_it a, int a_count, b_it b, int b_count, comp_t comp,
  int* lower, int* matches, int* starts, int* partitions,
  typename std::iterator_traits<a_it>::value_type* samples, int* partials,
  reduction_it join_count, context_t& context, hipEvent_t event = nullptr) {
  typedef typename scan_launch_default_t<int>::type_t_ scan_launch_t;
  int scan_nv = scan_launch_t::nv(context);
  // The search can add up the scan's partials when a tile of its needles
  // lies in two tiles of the scan at most.
  bool search_adds = a_count > scan_small_count &&
    search_launch_t::nv(context) <= scan_nv;
  if(a_count)
    sorted_search_launch<bounds_lower, search_launch_t>(a, a_count, b,
      b_count, lower, comp, partitions, samples, context, matches,
      search_adds ? partials : nullptr, scan_nv);
  if(search_adds)
    scan_finish<scan_type_exc, scan_launch_t>((const int*)matches, a_count,
      starts, plus_t<int>(), join_count, partials, context, event);
  else
    scan_launch<scan_type_exc, scan_launch_t>((const int*)matches, a_count,
      starts, plus_t<int>(), join_count, partials, context, event);
}

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
  // starts[i] = where the pairs of a[i] begin in the output.  The number of
  // pairs goes to pinned host memory (the output has to be allocated) and is
  // there once the event has passed, while the scan's last kernel still
  // runs.
  typedef typename conditional_typedef_t<launch_arg_t,
    detail::sorted_search_launch_default_t>::type_t search_launch_t;
  typedef typename std::iterator_traits<a_it>::value_type type_t;
  typedef typename detail::scan_launch_default_t<int>::type_t_ scan_launch_t;
  int nv = search_launch_t::nv(context);
  mem_t<int> lower(a_count, context), matches(a_count, context);
  mem_t<int> starts(a_count, context);
  mem_t<int> partitions(
    (size_t)div_up((int64_t)a_count + b_count, (int64_t)nv) + 1, context);
  mem_t<type_t> samples(
    detail::sorted_search_sample_count(a_count, b_count, nv), context);
  mem_t<int> partials(detail::scan_partials_count(a_count,
    scan_launch_t::nv(context)), context);
  mem_t<int> total(1, context, memory_space_host);
  const int* lower_data = lower.data();
  detail::join_count_launch<search_launch_t>(a, a_count, b, b_count, comp,
    lower.data(), matches.data(), starts.data(), partitions.data(),
    samples.data(), partials.data(), total.data(), context, context.event());
  hipError_t status = hipEventSynchronize(context.event());
  if(hipSuccess != status) throw cuda_exception_t(status);
  int join_count = total.data()[0];

  mem_t<int2> output(join_count, context);
  transform_lbs<launch_arg_t>(detail::join_pairs_f { output.data() },
    join_count, starts.data(), a_count, mgpu::make_tuple(lower_data),
    context);
  return output;
}

END_MGPU_NAMESPACE
