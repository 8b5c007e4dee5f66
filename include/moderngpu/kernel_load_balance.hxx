// mgpu for AMD CDNA4: load-balancing search over device-wide inputs.
//
//   transform_lbs(f, count, segments, num_segments, [cached iterators,]
//                 context, args...)
// calls f(index, seg, rank, [tuple of cached values,] args...) once for every
// work-item index in [0, count), where seg is the last segment whose start is
// <= index and rank = index - segments[seg].  Work is cut into tiles of equal
// size in (items + segments), so the cost per CTA does not depend on how the
// segment lengths are distributed.
//
// Interface after src/moderngpu/kernel_load_balance.hxx:8-86.
#pragma once
#include "cta_load_balance.hxx"
#include "search.hxx"

BEGIN_MGPU_NAMESPACE

namespace detail {

// Default tile for the search on gfx950: 256 threads (one wavefront per
// SIMD) x 16 items.
typedef launch_box_t<arch_gfx950_cta<256, 16, 16> > lbs_launch_default_t;

template<typename launch_t, typename func_t, typename segments_it,
  typename pointers_t, typename int_t>
struct transform_lbs_f {
  func_t f;
  int count;
  segments_it segments;
  int num_segments;
  pointers_t caching_iterators;
  const int_t* mp_data;

  template<typename... args_t>
  MGPU_DEVICE void operator()(int tid, int cta, args_t... args) const {
    typedef typename launch_t::sm_ptx params_t;
    enum { nt = params_t::nt, vt = params_t::vt, vt0 = params_t::vt0 };
    typedef cta_load_balance_t<nt, vt> load_balance_t;
    typedef cached_segment_load_t<nt, pointers_t> cached_load_t;
    typedef typename cached_load_t::value_t value_t;

    __shared__ struct {
      typename load_balance_t::storage_t lbs;
      typename cached_load_t::storage_t cached;
    } shared;

    auto lbs = load_balance_t().load_balance(count, segments, num_segments,
      tid, cta, mp_data, shared.lbs);

    // Items of the tile belong to segments [b_begin - 1, b_end).
    range_t seg_range { lbs.merge_range.b_begin - 1, lbs.merge_range.b_end };
    array_t<value_t, vt> cached_values = cached_load_t::template load<vt0>(
      tid, lbs.merge_range.a_count(), seg_range, lbs.segments,
      shared.cached, caching_iterators);

    strided_iterate<nt, vt, vt0>([&](int i, int) {
      f(lbs.indices[i], lbs.segments[i], lbs.ranks[i], cached_values[i],
        args...);
    }, tid, lbs.merge_range.a_count());
  }
};

} // namespace detail

namespace detail {

enum { lbs_phase_partition = 1, lbs_phase_tiles = 2, lbs_phase_all = 3 };

// Partition + tile kernels with the partition array in caller-provided
// device memory (div_up(count + num_segments, nv) + 1 ints).
template<typename launch_t, typename func_t, typename segments_it,
  typename pointers_t, typename... args_t>
void transform_lbs_launch(func_t f, int count, segments_it segments,
  int num_segments, pointers_t caching_iterators, int* mp_data, int phases,
  context_t& context, args_t... args) {

  if(count + num_segments <= 0) return;
  if(phases & lbs_phase_partition)
    load_balance_partitions_into((int64_t)count, segments, num_segments,
      launch_t::nv(context), mp_data, context);

  if(phases & lbs_phase_tiles) {
    transform_lbs_f<launch_t, func_t, segments_it, pointers_t, int>
      k { f, count, segments, num_segments, caching_iterators, mp_data };
    cta_transform<launch_t>(k, count + num_segments, context, args...);
  }
}

} // namespace detail

template<typename launch_arg_t = empty_t, typename func_t,
  typename segments_it, typename pointers_t, typename... args_t>
void transform_lbs(func_t f, int count, segments_it segments,
  int num_segments, pointers_t caching_iterators, context_t& context,
  args_t... args) {

  typedef typename conditional_typedef_t<launch_arg_t,
    detail::lbs_launch_default_t>::type_t launch_t;

  if(count + num_segments <= 0) return;
  int num_partitions = div_up(count + num_segments, launch_t::nv(context)) + 1;
  mem_t<int> mp(num_partitions, context);
  detail::transform_lbs_launch<launch_t>(f, count, segments, num_segments,
    caching_iterators, mp.data(), detail::lbs_phase_all, context, args...);
}

// Without cached values: f(index, seg, rank, args...).
template<typename launch_arg_t = empty_t, typename func_t,
  typename segments_it, typename... args_t>
void transform_lbs(func_t f, int count, segments_it segments,
  int num_segments, context_t& context, args_t... args) {

  transform_lbs<launch_arg_t>(
    [=]MGPU_DEVICE(int index, int seg, int rank, tuple<>, args_t... args) {
      f(index, seg, rank, args...);
    },
    count, segments, num_segments, tuple<>(), context, args...
  );
}

namespace detail {
template<typename output_it>
struct lbs_store_seg_f {
  output_it output;
  MGPU_DEVICE void operator()(int index, int seg, int) const {
    output[index] = seg;
  }
};
} // namespace detail

// output[index] = segment of work-item index.
template<typename launch_arg_t = empty_t, typename segments_it,
  typename output_it>
void load_balance_search(int count, segments_it segments,
  int num_segments, output_it output, context_t& context) {
  transform_lbs<launch_arg_t>(detail::lbs_store_seg_f<output_it> { output },
    count, segments, num_segments, context);
}

END_MGPU_NAMESPACE
