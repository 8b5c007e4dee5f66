// mgpu for AMD CDNA4: the launch front ends every kernel of the library goes
// through.  The entry points and their argument orders are those of
// src/moderngpu/transform.hxx:14-102:
//   cta_launch     a grid of CTAs, each thread runs f(tid, cta, args...)
//   cta_transform  the same, grid sized to cover `count` items at nv per CTA
//   transform      f(index, args...) once per index
// A launch the runtime rejects is thrown as cuda_exception_t.
#pragma once

#include <algorithm>
#include <random>
#include "launch_box.hxx"

BEGIN_MGPU_NAMESPACE

namespace detail {

// nt threads per CTA for this box on this device.
template<typename launch_box>
int box_threads(const context_t& context) {
  return launch_box::cta_dim(context.ptx_version()).nt;
}

// nt * vt items per CTA.
template<typename launch_box>
int box_items(const context_t& context) {
  return launch_box::cta_dim(context.ptx_version()).nv();
}

// One index per (thread, slot): the strided slots of CTA `cta`'s tile that
// lie below count.
template<typename launch_box>
struct transform_f {
  template<typename func_t, typename... args_t>
  MGPU_DEVICE void operator()(int tid, int cta, func_t f, size_t count,
    args_t... args) {
    typedef typename launch_box::sm_ptx params_t;
    int first = params_t::nt * params_t::vt * cta;
    int valid = (int)count - first;
    strided_iterate<params_t::nt, params_t::vt, params_t::vt0>(
      [&](int, int slot) { f(first + slot, args...); }, tid, valid);
  }
};

} // namespace detail

////////////////////////////////////////////////////////////////////////////////
// cta_launch.  An empty grid launches nothing.

template<typename launch_box, typename func_t, typename... args_t>
void cta_launch(func_t f, int num_ctas, context_t& context, args_t... args) {
  if(num_ctas < 1) return;
  auto kernel = launch_box_cta_k<launch_box, func_t, args_t...>;
  hipLaunchKernelGGL(kernel, dim3(num_ctas),
    dim3(detail::box_threads<launch_box>(context)), 0, context.stream(),
    f, num_ctas, args...);
  if(hipError_t status = hipGetLastError(); hipSuccess != status)
    throw cuda_exception_t(status);
}

// The tile count is only known on the device: a fixed grid of several CTAs per
// resident slot walks the tiles with a grid stride, and a CTA stops at the
// first tile index at or past *num_tiles.
namespace detail {
template<typename func_t>
struct strided_tiles_f {
  func_t f;
  const int* num_tiles;
  template<typename... args_t>
  MGPU_DEVICE void operator()(int tid, int cta, args_t... args) {
    for(int tile = cta, end = *num_tiles; tile < end; tile += (int)gridDim.x)
      f(tid, tile, args...);
  }
};
} // namespace detail

template<typename launch_box, typename func_t, typename... args_t>
void cta_launch(func_t f, const int* num_tiles, context_t& context,
  args_t... args) {
  detail::strided_tiles_f<func_t> strided { f, num_tiles };
  // Resident CTAs of the kernel that is launched (the walking one); a context
  // that does not fill in its device properties gets the count of compute
  // units from the runtime.
  int num_blocks = 0;
  hipError_t result = hipOccupancyMaxActiveBlocksPerMultiprocessor(
    &num_blocks,
    launch_box_cta_k<launch_box, detail::strided_tiles_f<func_t>, args_t...>,
    detail::box_threads<launch_box>(context), (size_t)0);
  if(hipSuccess != result) throw cuda_exception_t(result);
  int num_cus = context.props().multiProcessorCount;
  if(num_cus <= 0) {
    int device = 0;
    result = hipGetDevice(&device);
    if(hipSuccess == result)
      result = hipDeviceGetAttribute(&num_cus,
        hipDeviceAttributeMultiprocessorCount, device);
    if(hipSuccess != result) throw cuda_exception_t(result);
  }
  int grid = 8 * num_cus * num_blocks;
  // Nothing would run although *num_tiles may be positive.
  if(grid < 1) throw cuda_exception_t(hipErrorInvalidConfiguration);
  cta_launch<launch_box>(strided, grid, context, args...);
}

////////////////////////////////////////////////////////////////////////////////
// cta_transform: ceil(count / nv) CTAs.

template<typename launch_box, typename func_t, typename... args_t>
void cta_transform(func_t f, int count, context_t& context, args_t... args) {
  int num_ctas = div_up(count, detail::box_items<launch_box>(context));
  cta_launch<launch_box>(f, num_ctas, context, args...);
}

////////////////////////////////////////////////////////////////////////////////
// transform.

template<typename launch_box, typename func_t, typename... args_t>
void transform(func_t f, size_t count, context_t& context, args_t... args) {
  cta_transform<launch_box>(detail::transform_f<launch_box>(), (int)count,
    context, f, count, args...);
}

////////////////////////////////////////////////////////////////////////////////
// The <nt, vt> spellings: launch_params_t<nt, vt> as the box.

template<int nt, int vt = 1, typename func_t, typename... args_t>
void cta_launch(func_t f, int num_ctas, context_t& context, args_t... args) {
  cta_launch<launch_params_t<nt, vt> >(f, num_ctas, context, args...);
}
template<int nt, int vt = 1, typename func_t, typename... args_t>
void cta_transform(func_t f, int count, context_t& context, args_t... args) {
  cta_transform<launch_params_t<nt, vt> >(f, count, context, args...);
}
template<size_t nt = 128, int vt = 1, typename func_t, typename... args_t>
void transform(func_t f, size_t count, context_t& context, args_t... args) {
  transform<launch_params_t<nt, vt> >(f, count, context, args...);
}

END_MGPU_NAMESPACE
