// mgpu for AMD CDNA4: kernel launch front ends -- cta_launch (a grid of CTAs
// running f(tid, cta, args...)), cta_transform (grid sized from a work-item
// count) and transform (f(index, args...) per work-item).  Interface after
// src/moderngpu/transform.hxx:14-102.  Launch failures are reported as
// cuda_exception_t instead of being dropped.
#pragma once

#include <random>
#include <algorithm>
#include "launch_box.hxx"

BEGIN_MGPU_NAMESPACE

////////////////////////////////////////////////////////////////////////////////
// Launch num_ctas CTAs.  Nothing is launched for num_ctas == 0.

template<typename launch_box, typename func_t, typename... args_t>
void cta_launch(func_t f, int num_ctas, context_t& context, args_t... args) {
  cta_dim_t cta = launch_box::cta_dim(context.ptx_version());
  if(num_ctas <= 0) return;
  hipLaunchKernelGGL((launch_box_cta_k<launch_box, func_t, args_t...>),
    dim3(num_ctas), dim3(cta.nt), 0, context.stream(), f, num_ctas, args...);
  hipError_t result = hipGetLastError();
  if(hipSuccess != result) throw cuda_exception_t(result);
}

template<int nt, int vt = 1, typename func_t, typename... args_t>
void cta_launch(func_t f, int num_ctas, context_t& context, args_t... args) {
  cta_launch<launch_params_t<nt, vt> >(f, num_ctas, context, args...);
}

////////////////////////////////////////////////////////////////////////////////
// Launch enough CTAs to cover `count` work-items at nv = nt * vt per CTA.

template<typename launch_box, typename func_t, typename... args_t>
void cta_transform(func_t f, int count, context_t& context, args_t... args) {
  cta_dim_t cta = launch_box::cta_dim(context.ptx_version());
  cta_launch<launch_box>(f, div_up(count, cta.nv()), context, args...);
}

template<int nt, int vt = 1, typename func_t, typename... args_t>
void cta_transform(func_t f, int count, context_t& context, args_t... args) {
  cta_transform<launch_params_t<nt, vt> >(f, count, context, args...);
}

////////////////////////////////////////////////////////////////////////////////
// Persistent launch: a device-resident tile count, CTAs loop with a grid
// stride.  Every CTA leaves the loop once cta >= *num_tiles.

template<typename launch_box, typename func_t, typename... args_t>
void cta_launch(func_t f, const int* num_tiles, context_t& context,
  args_t... args) {
  // Oversubscribe the resident-CTA count to even out tile cost.
  int num_ctas = 8 * occupancy<launch_box>(f, context);
  auto k = [=]MGPU_DEVICE(int tid, int cta, args_t... args) {
    int count = *num_tiles;
    for(; cta < count; cta += num_ctas)
      f(tid, cta, args...);
  };
  cta_launch<launch_box>(k, num_ctas, context, args...);
}

////////////////////////////////////////////////////////////////////////////////
// transform: f(index, args...) for index in [0, count).

namespace detail {

template<typename launch_t>
struct transform_f {
  template<typename func_t, typename... args_t>
  MGPU_DEVICE void operator()(int tid, int cta, func_t f, size_t count,
    args_t... args) {
    typedef typename launch_t::sm_ptx params_t;
    enum { nt = params_t::nt, vt = params_t::vt, vt0 = params_t::vt0 };

    range_t range = get_tile(cta, nt * vt, (int)count);
    strided_iterate<nt, vt, vt0>([=](int i, int j) {
      f(range.begin + j, args...);
    }, tid, range.count());
  }
};

} // namespace detail

template<typename launch_t, typename func_t, typename... args_t>
void transform(func_t f, size_t count, context_t& context, args_t... args) {
  cta_transform<launch_t>(detail::transform_f<launch_t>(), (int)count,
    context, f, count, args...);
}

template<size_t nt = 128, int vt = 1, typename func_t, typename... args_t>
void transform(func_t f, size_t count, context_t& context, args_t... args) {
  transform<launch_params_t<nt, vt> >(f, count, context, args...);
}

END_MGPU_NAMESPACE
