// mgpu for AMD CDNA4 (gfx950): compile-time helpers and the function/lambda
// qualifier macros every other header uses.
// API surface follows moderngpu's meta.hxx (src/moderngpu/meta.hxx:11-238);
// the implementation is written for hipcc and 64-lane wavefronts.
#pragma once

#include <hip/hip_runtime.h>

#include <typeinfo>
#include <type_traits>
#include <iterator>
#include <cassert>
#include <cfloat>
#include <cstdint>
#include <cstddef>

#ifndef MGPU_HOST_DEVICE
  #define MGPU_HOST_DEVICE __forceinline__ __device__ __host__
#endif
#ifndef MGPU_DEVICE
  #define MGPU_DEVICE __device__
#endif
// hipcc accepts __host__ __device__ on lambdas, but keeping the macro
// device-only matches what callers written against moderngpu expect
// (meta.hxx:27-36 of the reference).
#ifndef MGPU_LAMBDA
  #define MGPU_LAMBDA __device__
#endif

#ifndef PRAGMA_UNROLL
  #define PRAGMA_UNROLL _Pragma("unroll")
#endif

#define BEGIN_MGPU_NAMESPACE namespace mgpu {
#define END_MGPU_NAMESPACE }

#define MGPU_ALIGN(x) __attribute__((aligned(x)))
#define MGPU_ALIGN_MAX __attribute__((aligned))

#ifndef M_PI
  #define M_PI 3.14159265358979323846
#endif

BEGIN_MGPU_NAMESPACE

template<bool B, class T = void>
using enable_if_t = typename std::enable_if<B, T>::type;

// A CDNA wavefront is 64 lanes.  The name is kept from the reference
// (meta.hxx:54, where it is 32) because user code sizes per-warp arrays by it.
enum { warp_size = 64 };

MGPU_HOST_DEVICE constexpr bool is_pow2(int x) { return 0 == (x & (x - 1)); }
MGPU_HOST_DEVICE constexpr int div_up(int x, int y) { return (x + y - 1) / y; }
MGPU_HOST_DEVICE constexpr int64_t div_up(int64_t x, int64_t y) {
  return (x + y - 1) / y;
}
MGPU_HOST_DEVICE constexpr size_t div_up(size_t x, size_t y) {
  return (x + y - 1) / y;
}
MGPU_HOST_DEVICE constexpr int s_log2(int x, int p = 0) {
  return x > 1 ? s_log2(x / 2) + 1 : p;
}
MGPU_HOST_DEVICE constexpr size_t s_log2(size_t x, size_t p = 0) {
  return x > 1 ? s_log2(x / 2) + 1 : p;
}

// Tie behaviour matters for bit-exact max/min of floats (+0/-0): the left
// operand wins ties, as in the reference (meta.hxx:113-120).
template<typename real_t>
MGPU_HOST_DEVICE constexpr real_t min(real_t a, real_t b) {
  return (b < a) ? b : a;
}
template<typename real_t>
MGPU_HOST_DEVICE constexpr real_t max(real_t a, real_t b) {
  return (a < b) ? b : a;
}

struct empty_t { };

template<typename... args_t>
MGPU_HOST_DEVICE void swallow(args_t...) { }

// inherit_t<A, B, C> derives from A::rebind<inherit_t<B, C>>: a linear chain
// of the launch-box "arch" policies (reference meta.hxx:127-135).
template<typename... base_v>
struct inherit_t;

template<typename base_t, typename... base_v>
struct inherit_t<base_t, base_v...> :
  base_t::template rebind<inherit_t<base_v...> > { };

template<typename base_t>
struct inherit_t<base_t> : base_t { };

// type_a unless it is empty_t, then type_b.
template<typename type_a, typename type_b>
struct conditional_typedef_t {
  typedef typename std::conditional<
    !std::is_same<type_a, empty_t>::value, type_a, type_b
  >::type type_t;
};

// __restrict__ on pointer kernel arguments only.
template<typename arg_t>
struct add_restrict { typedef arg_t type; };
template<typename arg_t>
struct add_restrict<arg_t*> { typedef arg_t* __restrict__ type; };

template<typename arg_t>
MGPU_HOST_DEVICE typename add_restrict<arg_t>::type make_restrict(arg_t x) {
  typename add_restrict<arg_t>::type y = x;
  return y;
}

////////////////////////////////////////////////////////////////////////////////
// iterate<count>(f): f(0) ... f(count - 1) with the index a compile-time
// constant after inlining, so register arrays indexed by it stay in VGPRs.

namespace detail {
template<int i, int count, bool valid = (i < count)>
struct iterate_t {
  template<typename func_t>
  MGPU_HOST_DEVICE static void eval(func_t f) {
    f(i);
    iterate_t<i + 1, count>::eval(f);
  }
};
template<int i, int count>
struct iterate_t<i, count, false> {
  template<typename func_t>
  MGPU_HOST_DEVICE static void eval(func_t) { }
};
} // namespace detail

template<int begin, int end, typename func_t>
MGPU_HOST_DEVICE void iterate(func_t f) {
  detail::iterate_t<begin, end>::eval(f);
}
template<int count, typename func_t>
MGPU_HOST_DEVICE void iterate(func_t f) {
  detail::iterate_t<0, count>::eval(f);
}

template<int count, typename type_t>
MGPU_HOST_DEVICE type_t reduce(const type_t(&x)[count]) {
  type_t y;
  iterate<count>([&](int i) { y = i ? x[i] + y : x[i]; });
  return y;
}

template<int count, typename type_t>
MGPU_HOST_DEVICE void fill(type_t(&x)[count], type_t val) {
  iterate<count>([&](int i) { x[i] = val; });
}

////////////////////////////////////////////////////////////////////////////////
// strided order: register i of thread tid maps to tile element nt * i + tid
// (coalesced across the wavefront).  thread order: vt * tid + i.

template<int nt, int vt, typename func_t>
MGPU_DEVICE void strided_iterate(func_t f, int tid) {
  iterate<vt>([=](int i) { f(i, nt * i + tid); });
}

// The first vt0 iterations run unguarded when the tile is known to hold at
// least nt * vt0 elements.
template<int nt, int vt, int vt0 = vt, typename func_t>
MGPU_DEVICE void strided_iterate(func_t f, int tid, int count) {
  if(vt0 > 1 && count >= nt * vt0) {
    strided_iterate<nt, vt0>(f, tid);
  } else {
    iterate<vt0>([=](int i) {
      int j = nt * i + tid;
      if(j < count) f(i, j);
    });
  }
  iterate<vt0, vt>([=](int i) {
    int j = nt * i + tid;
    if(j < count) f(i, j);
  });
}

template<int vt, typename func_t>
MGPU_DEVICE void thread_iterate(func_t f, int tid) {
  iterate<vt>([=](int i) { f(i, vt * tid + i); });
}

END_MGPU_NAMESPACE
