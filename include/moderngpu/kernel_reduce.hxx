// mgpu for AMD CDNA4: device-wide reduction.
//
//   reduce(input, count, reduction, op, context)
// stores input[0] op input[1] op ... op input[count - 1] to *reduction
// (device or host-mapped memory).  Nothing is stored for count == 0.  op must
// be associative; operands are folded left to right, so it need not be
// commutative.
//
// Two launches: one partial per tile (the scan's upsweep kernel: 16-byte
// strided loads, thread order through LDS), then one CTA folds the partials
// the same way.  Inputs of a few thousand items go to that CTA directly.
// Interface after src/moderngpu/kernel_reduce.hxx:11-68.
#pragma once
#include "kernel_scan.hxx"

BEGIN_MGPU_NAMESPACE

namespace detail {

// One CTA folds everything, nt * vt items per pass: 16-byte strided loads,
// thread order through LDS, the thread folds its vt items, the CTA folds the
// thread results in thread order, and the pass result is folded behind the
// running total.
template<int nt, int vt, typename input_it, typename output_it,
  typename type_t, typename op_t>
struct reduce_final_f {
  input_it input;
  int count;
  output_it reduction;
  op_t op;

  MGPU_DEVICE void operator()(int tid, int) const {
    enum { nv = nt * vt, W = chunk_width_t<type_t, vt>::value };
    typedef tile_layout_t<W> layout_t;
    typedef cta_reduce_t<nt, type_t> reduce_t;
    __shared__ struct {
      alignas(16) type_t values[layout_t::capacity(nv)];
      typename reduce_t::storage_t reduce;
    } shared;
    if(count <= 0) return;

    type_t total = type_t();
    for(int cur = 0; cur < count; cur += nv) {
      int n = min(count - cur, (int)nv);
      type_t x[vt];
      scan_load_tile<nt, vt>(input, cur, n, nv == n, tid, shared.values, x);
      int mine = min(max(n - vt * tid, 0), (int)vt);
      type_t scalar = x[0];
      PRAGMA_UNROLL
      for(int i = 1; i < vt; ++i)
        if(i < mine) scalar = op(scalar, x[i]);
      type_t pass = reduce_t().reduce(tid, scalar, shared.reduce,
        div_up(n, (int)vt), op, false);
      total = cur ? op(total, pass) : pass;     // thread 0 only
      __syncthreads();
    }
    if(!tid) *reduction = total;
  }
};

enum { reduce_final_nt = 1024, reduce_small_count = 16384 };

// Partials needed for `count` items in tiles of nv.
MGPU_HOST_DEVICE size_t reduce_partials_count(int64_t count, int nv) {
  return count > reduce_small_count ? (size_t)div_up(count, (int64_t)nv) : 0;
}

// The reduction with its temporaries in caller-provided device memory:
// reduce_partials_count(count, nv) values of type_t.
template<typename launch_t, typename input_it, typename output_it,
  typename type_t, typename op_t>
void reduce_launch(input_it input, int count, output_it reduction, op_t op,
  type_t* partials, context_t& context) {
  if(count <= 0) return;
  if(count <= reduce_small_count) {
    reduce_final_f<reduce_final_nt, spine_vt_t<type_t>::value, input_it,
      output_it, type_t, op_t>
      k { input, count, reduction, op };
    cta_launch<reduce_final_nt>(k, 1, context);
    return;
  }
  int num_tiles = div_up(count, launch_t::nv(context));
  scan_upsweep_f<launch_t, input_it, type_t, op_t>
    up { input, count, op, partials, num_tiles };
  cta_launch<launch_t>(up, xcd_grid(num_tiles), context);
  reduce_final_f<reduce_final_nt, spine_vt_t<type_t>::value, const type_t*,
    output_it, type_t, op_t>
    k { partials, num_tiles, reduction, op };
  cta_launch<reduce_final_nt>(k, 1, context);
}

} // namespace detail

template<typename launch_arg_t = empty_t, typename input_it,
  typename output_it, typename op_t>
void reduce(input_it input, int count, output_it reduction, op_t op,
  context_t& context) {

  if(detail::launcher_reduce<launch_arg_t>(input, count, reduction, op,
    context)) return;
  typedef typename std::iterator_traits<input_it>::value_type type_t;
  typedef typename conditional_typedef_t<launch_arg_t,
    typename detail::scan_launch_default_t<type_t>::type_t_>::type_t launch_t;

  mem_t<type_t> partials(detail::reduce_partials_count(count,
    launch_t::nv(context)), context);
  detail::reduce_launch<launch_t>(input, count, reduction, op,
    partials.data(), context);
}

// Reduction of f(index), index in [0, count); the value type is that of the
// output iterator.
template<typename launch_arg_t = empty_t, typename func_t,
  typename output_it, typename op_t>
void transform_reduce(func_t f, int count, output_it reduction, op_t op,
  context_t& context) {
  typedef typename std::iterator_traits<output_it>::value_type type_t;
  reduce<launch_arg_t>(make_load_iterator<type_t>(f), count, reduction, op,
    context);
}

END_MGPU_NAMESPACE
