// mgpu for AMD CDNA4 (gfx950): the qualifier macros every other header uses
// and the compile-time helpers (unrolled iteration, the launch-box inheritance
// chain, small constexpr arithmetic).  The public names are those of
// src/moderngpu/meta.hxx:11-238 so that code written against that library
// compiles; this is hipcc-only C++17 for 64-lane wavefronts.
#pragma once

#include <hip/hip_runtime.h>

#include <cassert>
#include <cfloat>
#include <cstddef>
#include <cstdint>
#include <iterator>
#include <type_traits>
#include <typeinfo>
#include <utility>

////////////////////////////////////////////////////////////////////////////////
// Qualifiers.  MGPU_LAMBDA stays device-only: callers written against
// moderngpu mark their lambdas with it and expect exactly that.

#ifndef MGPU_DEVICE
  #define MGPU_DEVICE __device__
#endif
#ifndef MGPU_HOST_DEVICE
  #define MGPU_HOST_DEVICE __forceinline__ __device__ __host__
#endif
#ifndef MGPU_LAMBDA
  #define MGPU_LAMBDA __device__
#endif
#ifndef M_PI
  #define M_PI 3.14159265358979323846
#endif

#ifndef PRAGMA_UNROLL
  #define PRAGMA_UNROLL _Pragma("unroll")
#endif

#define MGPU_ALIGN(bytes) __attribute__((aligned(bytes)))

#define BEGIN_MGPU_NAMESPACE namespace mgpu {
#define END_MGPU_NAMESPACE }

BEGIN_MGPU_NAMESPACE

// Lanes of a wavefront.  moderngpu calls this warp_size (32 there); code that
// sizes per-warp arrays or masks by the constant adapts by itself.
enum { warp_size = 64 };

// The "no argument given" placeholder of launch-box and tuple parameters.
struct empty_t { };

template<bool condition, class type_t = void>
using enable_if_t = typename std::enable_if<condition, type_t>::type;

////////////////////////////////////////////////////////////////////////////////
// constexpr arithmetic

// ceil(x / y) for non-negative x and positive y, in the three index widths
// the library uses (plain overloads, so enumerators and mixed int arguments
// convert).  The int form adds in unsigned arithmetic: x + y - 1 may pass
// 2^31 for item counts close to the index limit.
MGPU_HOST_DEVICE constexpr int div_up(int x, int y) {
  return (int)(((unsigned)x + (unsigned)y - 1u) / (unsigned)y);
}
#define MGPU_DIV_UP(int_t)                                                    \
  MGPU_HOST_DEVICE constexpr int_t div_up(int_t x, int_t y) {                 \
    return (x + y - 1) / y;                                                   \
  }
MGPU_DIV_UP(int64_t) MGPU_DIV_UP(size_t)
#undef MGPU_DIV_UP
MGPU_HOST_DEVICE constexpr bool is_pow2(int x) { return !(x & (x - 1)); }

// floor(log2 x) for x >= 1.
template<typename int_t>
MGPU_HOST_DEVICE constexpr int_t s_log2(int_t x, int_t sum = 0) {
  return x < 2 ? sum : s_log2(x >> 1, sum + 1);
}

// Ties go to the left operand: max(+0.f, -0.f) is +0.f, max(-0.f, +0.f) is
// -0.f, and max/min reductions of floats are bit-for-bit what a serial loop
// with these functions produces.
template<typename real_t>
MGPU_HOST_DEVICE constexpr real_t max(real_t a, real_t b) {
  return (a < b) ? b : a;
}
template<typename real_t>
MGPU_HOST_DEVICE constexpr real_t min(real_t a, real_t b) {
  return (b < a) ? b : a;
}

// Takes any arguments and does nothing: swallow(f(args)...) evaluates a pack
// expansion for its side effects.
template<typename... args_t>
MGPU_HOST_DEVICE void swallow(args_t...) { }

////////////////////////////////////////////////////////////////////////////////
// Launch-box plumbing.

// inherit_t<A, B, C> is A rebased onto B rebased onto C: each architecture
// entry of a launch box derives from the entries listed after it, so a lookup
// of sm_XX finds the nearest one that is defined.
template<typename... base_v>
struct inherit_t;
template<typename last_t>
struct inherit_t<last_t> : last_t { };
template<typename first_t, typename... rest_v>
struct inherit_t<first_t, rest_v...> :
  first_t::template rebind<inherit_t<rest_v...> > { };

// type_a if the caller gave one, else the library's default type_b.
template<typename type_a, typename type_b>
struct conditional_typedef_t {
  typedef typename std::conditional<std::is_same<type_a, empty_t>::value,
    type_b, type_a>::type type_t;
};

// Kernel arguments that are plain pointers are passed on as __restrict__.
template<typename arg_t>
struct add_restrict {
  typedef arg_t type;
};
template<typename pointee_t>
struct add_restrict<pointee_t*> {
  typedef pointee_t* __restrict__ type;
};
template<typename arg_t>
MGPU_HOST_DEVICE typename add_restrict<arg_t>::type make_restrict(arg_t x) {
  return (typename add_restrict<arg_t>::type)x;
}

////////////////////////////////////////////////////////////////////////////////
// iterate<count>(f) calls f(0) ... f(count - 1); iterate<begin, end>(f) calls
// f(begin) ... f(end - 1).  The calls are a fold over an integer pack, so after
// inlining every index is a constant and register arrays indexed by it stay in
// VGPRs.

namespace detail {
template<int first, typename func_t, int... offset>
MGPU_HOST_DEVICE void iterate_pack(func_t& f,
  std::integer_sequence<int, offset...>) {
  (f(first + offset), ...);
}
} // namespace detail

template<int begin, int end, typename func_t>
MGPU_HOST_DEVICE void iterate(func_t f) {
  detail::iterate_pack<begin>(f,
    std::make_integer_sequence<int, (end > begin ? end - begin : 0)>());
}
template<int count, typename func_t>
MGPU_HOST_DEVICE void iterate(func_t f) {
  iterate<0, count>(f);
}

// Sum of a small array, and the same value into each of its elements.
template<int count, typename type_t>
MGPU_HOST_DEVICE type_t reduce(const type_t (&x)[count]) {
  type_t sum = x[0];
  PRAGMA_UNROLL
  for(int i = 1; i < count; ++i) sum = x[i] + sum;
  return sum;
}
template<int count, typename type_t>
MGPU_HOST_DEVICE void fill(type_t (&x)[count], type_t value) {
  PRAGMA_UNROLL
  for(int i = 0; i < count; ++i) x[i] = value;
}

////////////////////////////////////////////////////////////////////////////////
// A thread's vt slots of an nt * vt tile, f(i, slot):
//   strided order  slot = nt * i + tid   (coalesced across the wavefront)
//   thread order   slot = vt * tid + i   (contiguous per lane)
// With a count, slots at or past it are skipped; the first vt0 strided slots
// of a tile known to hold nt * vt0 elements are not even tested.

template<int nt, int vt, typename func_t>
MGPU_DEVICE void strided_iterate(func_t f, int tid) {
  iterate<vt>([&](int i) { f(i, nt * i + tid); });
}

template<int nt, int vt, int vt0 = vt, typename func_t>
MGPU_DEVICE void strided_iterate(func_t f, int tid, int count) {
  bool full_rows = vt0 > 1 && count >= nt * vt0;
  iterate<vt>([&](int i) {
    int slot = nt * i + tid;
    if((full_rows && i < vt0) || slot < count) f(i, slot);
  });
}

template<int vt, typename func_t>
MGPU_DEVICE void thread_iterate(func_t f, int tid) {
  iterate<vt>([&](int i) { f(i, vt * tid + i); });
}

END_MGPU_NAMESPACE
