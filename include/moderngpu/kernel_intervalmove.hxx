// mgpu for AMD CDNA4: interval expand / gather / scatter / move, all thin
// functors over transform_lbs (interface after
// src/moderngpu/kernel_intervalmove.hxx:7-65).
#pragma once
#include "kernel_load_balance.hxx"

BEGIN_MGPU_NAMESPACE

namespace detail {
// output[index] = value of the item's segment, for any output iterator ...
template<typename type_t, typename output_it>
struct interval_expand_f {
  output_it output;
  MGPU_DEVICE void operator()(int index, int, int,
    tuple<type_t> desc) const {
    output[index] = get<0>(desc);
  }
};
// ... and, for pointers, W values per call written with the widest stores
// the element type allows.
template<typename type_t>
struct interval_expand_f<type_t, type_t*> {
  typedef void chunk_functor_tag;
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
} // namespace detail

// output[index] = input[segment of index]: each per-segment value is
// replicated over the segment's items.
template<typename launch_arg_t = empty_t, typename input_it,
  typename segments_it, typename output_it>
void interval_expand(input_it input, int count, segments_it segments,
  int num_segments, output_it output, context_t& context) {

  typedef typename std::iterator_traits<input_it>::value_type type_t;
  transform_lbs<launch_arg_t>(
    detail::interval_expand_f<type_t, output_it> { output },
    count, segments, num_segments, make_tuple(input), context);
}

// output[index] = input[gather[seg] + rank].
template<typename launch_arg_t = empty_t, typename input_it,
  typename segments_it, typename gather_it, typename output_it>
void interval_gather(input_it input, int count, segments_it segments,
  int num_segments, gather_it gather, output_it output, context_t& context) {

  transform_lbs<launch_arg_t>(
    []MGPU_DEVICE(int index, int, int rank, tuple<int> desc,
      input_it input, output_it output) {
      output[index] = input[get<0>(desc) + rank];
    },
    count, segments, num_segments, make_tuple(gather), context, input, output
  );
}

// output[scatter[seg] + rank] = input[index].
template<typename launch_arg_t = empty_t, typename input_it,
  typename segments_it, typename scatter_it, typename output_it>
void interval_scatter(input_it input, int count, segments_it segments,
  int num_segments, scatter_it scatter, output_it output,
  context_t& context) {

  transform_lbs<launch_arg_t>(
    []MGPU_DEVICE(int index, int, int rank, tuple<int> desc,
      input_it input, output_it output) {
      output[get<0>(desc) + rank] = input[index];
    },
    count, segments, num_segments, make_tuple(scatter), context, input, output
  );
}

// output[scatter[seg] + rank] = input[gather[seg] + rank].
template<typename launch_arg_t = empty_t,
  typename input_it, typename segments_it, typename scatter_it,
  typename gather_it, typename output_it>
void interval_move(input_it input, int count, segments_it segments,
  int num_segments, scatter_it scatter, gather_it gather, output_it output,
  context_t& context) {

  transform_lbs<launch_arg_t>(
    []MGPU_DEVICE(int, int, int rank, tuple<int, int> desc,
      input_it input, output_it output) {
      output[get<0>(desc) + rank] = input[get<1>(desc) + rank];
    },
    count, segments, num_segments, make_tuple(scatter, gather), context,
    input, output
  );
}

END_MGPU_NAMESPACE
