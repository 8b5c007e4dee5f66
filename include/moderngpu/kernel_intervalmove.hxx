// mgpu for AMD CDNA4: the interval functions.  Each is transform_lbs with a
// functor that copies one item; the per-segment values (fill value, gather
// base, scatter base) travel as the cached tuple.  Signatures after
// src/moderngpu/kernel_intervalmove.hxx:7-65.
#pragma once
#include "kernel_load_balance.hxx"

BEGIN_MGPU_NAMESPACE

namespace detail {
// output[index] = value of the item's segment, for any output iterator ...
template<typename type_t, typename output_it, typename enable_t = void>
struct interval_expand_f {
  output_it output;
  MGPU_DEVICE void operator()(int index, int, int,
    tuple<type_t> desc) const {
    output[index] = get<0>(desc);
  }
};
// ... for pointers to elements of 16 bytes or more the same, one element per
// lane and store (consecutive lanes then write consecutive 16-byte pieces;
// four elements per lane would have every store touch a quarter of each cache
// line: 2^28 16-byte elements 1,300 us against 904 us) ...
template<typename type_t>
struct interval_expand_f<type_t, type_t*,
  typename std::enable_if<(sizeof(type_t) >= 16)>::type> {
  enum { lbs_tiles_per_cta = 2 };
  type_t* output;
  MGPU_DEVICE void operator()(int index, int, int,
    tuple<type_t> desc) const {
    output[index] = get<0>(desc);
  }
};
// ... and, for pointers to smaller elements, W values per call written with
// the widest stores the element type allows.
template<typename type_t>
struct interval_expand_f<type_t, type_t*,
  typename std::enable_if<(sizeof(type_t) < 16)>::type> {
  typedef void chunk_functor_tag;
  enum { lbs_tiles_per_cta = 2 };   // two reads, then only stores: see
                                    // lbs_tiles_per_cta_t
  type_t* output;
  MGPU_DEVICE void operator()(int index, int, int,
    tuple<type_t> desc) const {
    output[index] = get<0>(desc);
  }
  template<int W>
  MGPU_DEVICE void chunk(int index, const int (&)[W], const int (&)[W],
    const tuple<type_t> (&desc)[W]) const {
    type_t x[W];
    PRAGMA_UNROLL
    for(int e = 0; e < W; ++e) x[e] = get<0>(desc[e]);
    store_consecutive<W>(output + index, x);
  }
};

// One item of gather / scatter / move.  The segment's tuple holds the scatter
// base (if scattering) followed by the gather base (if gathering); an item
// that is neither gathered nor scattered sits at its own index.
template<bool scatters, bool gathers, typename input_it, typename output_it>
struct interval_copy_f {
  input_it input;
  output_it output;
  template<typename bases_t>
  MGPU_DEVICE void operator()(int index, int, int rank, bases_t bases) const {
    int from = index, to = index;
    if constexpr(scatters) to = get<0>(bases) + rank;
    if constexpr(gathers) from = get<scatters ? 1 : 0>(bases) + rank;
    output[to] = input[from];
  }
};

// Pointer to pointer: W consecutive items per call.  All W loads are issued
// before the first store, and the side that is not gathered or scattered
// moves as one 16-byte (or wider) access.
template<bool scatters, bool gathers, typename type_t>
struct interval_copy_chunks_f {
  typedef void chunk_functor_tag;
  const type_t* input;
  type_t* output;

  template<typename bases_t>
  MGPU_DEVICE void operator()(int index, int, int rank, bases_t bases) const {
    int from = index, to = index;
    if constexpr(scatters) to = get<0>(bases) + rank;
    if constexpr(gathers) from = get<scatters ? 1 : 0>(bases) + rank;
    output[to] = input[from];
  }

  // Gathered elements are loaded one by one (W independent loads; measured
  // faster than testing for a chunk that lies in one segment).  Scattered
  // elements of one segment are consecutive and go out as one store -- W
  // single stores per lane would each write a quarter of every cache line
  // they touch -- and element by element when the chunk crosses a segment
  // boundary.
  template<int W, typename bases_t>
  MGPU_DEVICE void chunk(int index, const int (&seg)[W], const int (&rank)[W],
    const bases_t (&bases)[W]) const {
    bool one_segment = seg[0] == seg[W - 1];
    type_t x[W];
    if constexpr(gathers) {
      PRAGMA_UNROLL
      for(int e = 0; e < W; ++e)
        x[e] = input[get<scatters ? 1 : 0>(bases[e]) + rank[e]];
    } else
      load_consecutive<W>(input + index, x);
    if constexpr(scatters) {
      if(one_segment)
        store_consecutive<W>(output + get<0>(bases[0]) + rank[0], x);
      else {
        PRAGMA_UNROLL
        for(int e = 0; e < W; ++e) output[get<0>(bases[e]) + rank[e]] = x[e];
      }
    } else
      store_consecutive<W>(output + index, x);
  }
};

// The functor for a pair of iterator types.
template<bool scatters, bool gathers, typename input_it, typename output_it>
struct interval_copy_select_t {
  typedef interval_copy_f<scatters, gathers, input_it, output_it> type;
};
// Pointers to elements of less than 16 bytes: W elements per lane.  (Wider
// elements go one per lane, as in interval_expand_f.)
template<bool scatters, bool gathers, typename type_t>
struct interval_copy_select_t<scatters, gathers, const type_t*, type_t*> {
  typedef typename std::conditional<(sizeof(type_t) < 16),
    interval_copy_chunks_f<scatters, gathers, type_t>,
    interval_copy_f<scatters, gathers, const type_t*, type_t*> >::type type;
};
template<bool scatters, bool gathers, typename type_t>
struct interval_copy_select_t<scatters, gathers, type_t*, type_t*> {
  typedef typename std::conditional<(sizeof(type_t) < 16),
    interval_copy_chunks_f<scatters, gathers, type_t>,
    interval_copy_f<scatters, gathers, type_t*, type_t*> >::type type;
};

} // namespace detail

// Segment s's one value written to each of its items:
// output[i] = input[segment of i].
template<typename launch_arg_t = empty_t, typename input_it,
  typename segments_it, typename output_it>
void interval_expand(input_it input, int count, segments_it segments,
  int num_segments, output_it output, context_t& context) {
  if(detail::launcher_interval<launch_arg_t>(input, count, segments,
    num_segments, empty_t(), empty_t(), output, context)) return;
  typedef typename std::iterator_traits<input_it>::value_type type_t;
  detail::interval_expand_f<type_t, output_it> fill { output };
  transform_lbs<launch_arg_t>(fill, count, segments, num_segments,
    mgpu::make_tuple(input), context);
}

// Segment s reads its items from input starting at gather[s]:
// output[i] = input[gather[s] + rank of i].
template<typename launch_arg_t = empty_t, typename input_it,
  typename segments_it, typename gather_it, typename output_it>
void interval_gather(input_it input, int count, segments_it segments,
  int num_segments, gather_it gather, output_it output, context_t& context) {
  if(detail::launcher_interval<launch_arg_t>(input, count, segments,
    num_segments, empty_t(), gather, output, context)) return;
  typename detail::interval_copy_select_t<false, true, input_it,
    output_it>::type copy { input, output };
  transform_lbs<launch_arg_t>(copy, count, segments, num_segments,
    mgpu::make_tuple(gather), context);
}

// Segment s writes its items to output starting at scatter[s]:
// output[scatter[s] + rank of i] = input[i].
template<typename launch_arg_t = empty_t, typename input_it,
  typename segments_it, typename scatter_it, typename output_it>
void interval_scatter(input_it input, int count, segments_it segments,
  int num_segments, scatter_it scatter, output_it output,
  context_t& context) {
  if(detail::launcher_interval<launch_arg_t>(input, count, segments,
    num_segments, scatter, empty_t(), output, context)) return;
  typename detail::interval_copy_select_t<true, false, input_it,
    output_it>::type copy { input, output };
  transform_lbs<launch_arg_t>(copy, count, segments, num_segments,
    mgpu::make_tuple(scatter), context);
}

// Both at once: output[scatter[s] + rank] = input[gather[s] + rank].
template<typename launch_arg_t = empty_t,
  typename input_it, typename segments_it, typename scatter_it,
  typename gather_it, typename output_it>
void interval_move(input_it input, int count, segments_it segments,
  int num_segments, scatter_it scatter, gather_it gather, output_it output,
  context_t& context) {
  if(detail::launcher_interval<launch_arg_t>(input, count, segments,
    num_segments, scatter, gather, output, context)) return;
  typename detail::interval_copy_select_t<true, true, input_it,
    output_it>::type copy { input, output };
  transform_lbs<launch_arg_t>(copy, count, segments, num_segments,
    mgpu::make_tuple(scatter, gather), context);
}

END_MGPU_NAMESPACE
