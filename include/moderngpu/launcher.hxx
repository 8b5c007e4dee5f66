// mgpu for AMD CDNA4: dispatch from the public templates to the prebuilt
// kernels of libmgpu_hip.so.
//
// By default every public template instantiates its kernels in the caller's
// translation unit (the library is header-only, like the CUDA library whose
// interface it mirrors).  A caller that defines MGPU_HIP_LAUNCHER before
// including these headers and links libmgpu_hip.so gets, for the argument
// combinations the extern "C" layer covers -- raw pointers, value types
// {int, unsigned, 64-bit ints, float, double}, operators plus_t / maximum_t /
// minimum_t (segreduce, scan, reduce; spmv on float / double), element sizes
// 1/2/4/8/16 bytes for the interval functions, no explicit launch box -- a
// call into that layer instead: the same kernels, compiled once, and nothing
// of them in the caller's object code.  Everything
// else (functors, iterators, user types and operators, explicit launch boxes)
// still instantiates in place.  Temporaries come from context.alloc() and the
// launches go to context.stream(), as in the header-only path; a non-zero
// return code of the layer is thrown as cuda_exception_t.
//
// Each helper below returns true when it has made the call.
#pragma once
#include <cstdio>
#include <cstdlib>
#include "context.hxx"
#include "memory.hxx"
#include "operators.hxx"

#ifdef MGPU_HIP_LAUNCHER
#include "../mgpu_hip.h"
#endif

BEGIN_MGPU_NAMESPACE

namespace detail {

#ifdef MGPU_HIP_LAUNCHER

template<typename type_t> struct launcher_dtype_t { enum { value = -1 }; };
#define MGPU_LAUNCHER_DTYPE(type, code)                                       \
  template<> struct launcher_dtype_t<type> { enum { value = code }; };
MGPU_LAUNCHER_DTYPE(int, MGPU_I32)
MGPU_LAUNCHER_DTYPE(unsigned, MGPU_U32)
MGPU_LAUNCHER_DTYPE(long, MGPU_I64)
MGPU_LAUNCHER_DTYPE(long long, MGPU_I64)
MGPU_LAUNCHER_DTYPE(unsigned long, MGPU_U64)
MGPU_LAUNCHER_DTYPE(unsigned long long, MGPU_U64)
MGPU_LAUNCHER_DTYPE(float, MGPU_F32)
MGPU_LAUNCHER_DTYPE(double, MGPU_F64)
#undef MGPU_LAUNCHER_DTYPE
static_assert(8 == sizeof(long), "MGPU_I64 / MGPU_U64 stand for long");

// Operator code, for the operator on exactly the value type.
template<typename op_t, typename type_t>
struct launcher_op_t { enum { value = -1 }; };
template<typename type_t>
struct launcher_op_t<plus_t<type_t>, type_t> { enum { value = MGPU_PLUS }; };
template<typename type_t>
struct launcher_op_t<maximum_t<type_t>, type_t> {
  enum { value = MGPU_MAXIMUM };
};
template<typename type_t>
struct launcher_op_t<minimum_t<type_t>, type_t> {
  enum { value = MGPU_MINIMUM };
};

// it_t is `type_t*` or `const type_t*` (writable: `type_t*` only).
template<typename it_t, typename type_t, bool writable = false>
struct launcher_points_to_t {
  typedef typename std::remove_pointer<it_t>::type pointee_t;
  enum {
    value = std::is_pointer<it_t>::value &&
      std::is_same<typename std::remove_cv<pointee_t>::type, type_t>::value &&
      (!writable || !std::is_const<pointee_t>::value)
  };
};

template<typename type_t>
struct launcher_elem_bytes_t {
  enum {
    size = (int)sizeof(type_t),
    value = std::is_trivially_copyable<type_t>::value &&
      (1 == size || 2 == size || 4 == size || 8 == size || 16 == size) &&
      (int)alignof(type_t) >= size    // the layer moves naturally aligned words
  };
};

inline void launcher_check(int code) {
  if(code) throw cuda_exception_t((hipError_t)code);
}

// Number of calls that went to the library (for tests).  With the environment
// variable MGPU_HIP_LAUNCHER_REPORT set, a program built with
// MGPU_HIP_LAUNCHER prints the count to stderr when it ends ("mgpu launcher
// calls: N", also when N is 0), and a line when the first call is made (a
// program that is ended from outside never gets to the other): that is how a
// program that cannot be edited -- one written for the CUDA library and only
// recompiled -- shows which way its calls went.
struct launcher_counter_t {
  long calls = 0;
  ~launcher_counter_t() {
    if(getenv("MGPU_HIP_LAUNCHER_REPORT"))
      fprintf(stderr, "mgpu launcher calls: %ld\n", calls);
  }
};
inline long& launcher_calls() {
  static launcher_counter_t counter;
  return counter.calls;
}
inline void launcher_count_call() {
  long& calls = launcher_calls();
  if(!calls++ && getenv("MGPU_HIP_LAUNCHER_REPORT"))
    fprintf(stderr, "mgpu launcher: first call\n");
}
#ifdef MGPU_HIP_LAUNCHER
// The counter exists from program start in a build with the dispatch layer,
// so that its report at exit is printed whether or not a call went there.
static long* const launcher_counter_from_start = &launcher_calls();
#endif

template<typename launch_arg_t, typename input_it, typename segments_it,
  typename output_it, typename op_t, typename type_t>
bool launcher_segreduce(input_it input, int count, segments_it segments,
  int num_segments, output_it output, op_t, type_t init,
  context_t& context) {
  if constexpr(std::is_same<launch_arg_t, empty_t>::value &&
    launcher_dtype_t<type_t>::value >= 0 &&
    launcher_op_t<op_t, type_t>::value >= 0 &&
    launcher_points_to_t<input_it, type_t>::value &&
    launcher_points_to_t<segments_it, int>::value &&
    launcher_points_to_t<output_it, type_t, true>::value) {
    int dtype = launcher_dtype_t<type_t>::value;
    size_t bytes = mgpu_hip_segreduce_workspace_bytes(count, num_segments,
      dtype);
    mem_t<char> workspace(bytes, context);
    launcher_check(mgpu_hip_segreduce(input, count, segments, num_segments,
      output, dtype, launcher_op_t<op_t, type_t>::value, &init,
      workspace.data(), bytes, context.stream()));
    launcher_count_call();
    return true;
  } else
    return false;
}

template<typename launch_arg_t, typename matrix_it, typename columns_it,
  typename vector_it, typename segments_it, typename output_it>
bool launcher_spmv(matrix_it matrix, columns_it columns, vector_it vector,
  int count, segments_it segments, int num_segments, output_it output,
  context_t& context) {
  typedef typename std::iterator_traits<matrix_it>::value_type type_t;
  if constexpr(std::is_same<launch_arg_t, empty_t>::value &&
    (std::is_same<type_t, float>::value ||
      std::is_same<type_t, double>::value) &&
    launcher_points_to_t<matrix_it, type_t>::value &&
    launcher_points_to_t<columns_it, int>::value &&
    launcher_points_to_t<vector_it, type_t>::value &&
    launcher_points_to_t<segments_it, int>::value &&
    launcher_points_to_t<output_it, type_t, true>::value) {
    int dtype = launcher_dtype_t<type_t>::value;
    size_t bytes = mgpu_hip_segreduce_workspace_bytes(count, num_segments,
      dtype);
    mem_t<char> workspace(bytes, context);
    launcher_check(mgpu_hip_spmv(matrix, columns, vector, count, segments,
      num_segments, output, dtype, workspace.data(), bytes,
      context.stream()));
    launcher_count_call();
    return true;
  } else
    return false;
}

template<typename launch_arg_t, typename segments_it, typename output_it>
bool launcher_load_balance_search(int count, segments_it segments,
  int num_segments, output_it output, context_t& context) {
  if constexpr(std::is_same<launch_arg_t, empty_t>::value &&
    launcher_points_to_t<segments_it, int>::value &&
    launcher_points_to_t<output_it, int, true>::value) {
    size_t bytes = mgpu_hip_lbs_workspace_bytes(count, num_segments);
    mem_t<char> workspace(bytes, context);
    launcher_check(mgpu_hip_load_balance_search(count, segments,
      num_segments, output, workspace.data(), bytes, context.stream()));
    launcher_count_call();
    return true;
  } else
    return false;
}

// interval_expand / gather / scatter / move: `scatter` and `gather` are
// const int* or absent (empty_t).
template<typename launch_arg_t, typename input_it, typename segments_it,
  typename scatter_it, typename gather_it, typename output_it>
bool launcher_interval(input_it input, int count,
  segments_it segments, int num_segments, scatter_it scatter,
  gather_it gather, output_it output, context_t& context) {
  typedef typename std::iterator_traits<input_it>::value_type type_t;
  enum {
    scatters = !std::is_same<scatter_it, empty_t>::value,
    gathers = !std::is_same<gather_it, empty_t>::value
  };
  if constexpr(std::is_same<launch_arg_t, empty_t>::value &&
    launcher_elem_bytes_t<type_t>::value &&
    launcher_points_to_t<input_it, type_t>::value &&
    launcher_points_to_t<segments_it, int>::value &&
    (!scatters || launcher_points_to_t<scatter_it, int>::value) &&
    (!gathers || launcher_points_to_t<gather_it, int>::value) &&
    launcher_points_to_t<output_it, type_t, true>::value) {
    int size = (int)sizeof(type_t);
    size_t bytes = mgpu_hip_lbs_workspace_bytes(count, num_segments);
    mem_t<char> workspace(bytes, context);
    void* ws = workspace.data();
    hipStream_t stream = context.stream();
    int code;
    if constexpr(scatters && gathers)
      code = mgpu_hip_interval_move(input, size, count, segments,
        num_segments, scatter, gather, output, ws, bytes, stream);
    else if constexpr(scatters)
      code = mgpu_hip_interval_scatter(input, size, count, segments,
        num_segments, scatter, output, ws, bytes, stream);
    else if constexpr(gathers)
      code = mgpu_hip_interval_gather(input, size, count, segments,
        num_segments, gather, output, ws, bytes, stream);
    else
      code = mgpu_hip_interval_expand(input, size, count, segments,
        num_segments, output, ws, bytes, stream);
    launcher_check(code);
    launcher_count_call();
    return true;
  } else
    return false;
}

// scan / scan_event without an event; the fold goes to a type_t* or is
// discarded.
template<typename launch_arg_t, typename input_it, typename output_it,
  typename op_t, typename reduction_it>
bool launcher_scan(bool inclusive, input_it input, int count,
  output_it output, op_t, reduction_it reduction, context_t& context,
  hipEvent_t event) {
  typedef typename std::iterator_traits<input_it>::value_type type_t;
  enum { discards =
    std::is_same<reduction_it, discard_iterator_t<type_t> >::value };
  if constexpr(std::is_same<launch_arg_t, empty_t>::value &&
    launcher_dtype_t<type_t>::value >= 0 &&
    launcher_op_t<op_t, type_t>::value >= 0 &&
    launcher_points_to_t<input_it, type_t>::value &&
    launcher_points_to_t<output_it, type_t, true>::value &&
    (discards || launcher_points_to_t<reduction_it, type_t, true>::value)) {
    if(event) return false;         // the layer cannot record one mid-call
    int dtype = launcher_dtype_t<type_t>::value;
    size_t bytes = mgpu_hip_scan_workspace_bytes(count, dtype);
    mem_t<char> workspace(bytes, context);
    void* total = nullptr;
    if constexpr(!discards) total = reduction;
    launcher_check(mgpu_hip_scan(input, count, output, dtype,
      launcher_op_t<op_t, type_t>::value, (int)inclusive, total,
      workspace.data(), bytes, context.stream()));
    launcher_count_call();
    return true;
  } else
    return false;
}

template<typename launch_arg_t, typename input_it, typename output_it,
  typename op_t>
bool launcher_reduce(input_it input, int count, output_it reduction, op_t,
  context_t& context) {
  typedef typename std::iterator_traits<input_it>::value_type type_t;
  if constexpr(std::is_same<launch_arg_t, empty_t>::value &&
    launcher_dtype_t<type_t>::value >= 0 &&
    launcher_op_t<op_t, type_t>::value >= 0 &&
    launcher_points_to_t<input_it, type_t>::value &&
    launcher_points_to_t<output_it, type_t, true>::value) {
    int dtype = launcher_dtype_t<type_t>::value;
    size_t bytes = mgpu_hip_reduce_workspace_bytes(count, dtype);
    mem_t<char> workspace(bytes, context);
    launcher_check(mgpu_hip_reduce(input, count, reduction, dtype,
      launcher_op_t<op_t, type_t>::value, workspace.data(), bytes,
      context.stream()));
    launcher_count_call();
    return true;
  } else
    return false;
}

// sorted_search on int keys ordered by less_t<int>.
template<typename launch_arg_t, typename needles_it, typename haystack_it,
  typename indices_it, typename comp_t>
bool launcher_sorted_search(bool upper, needles_it needles, int num_needles,
  haystack_it haystack, int num_haystack, indices_it indices, comp_t,
  context_t& context) {
  if constexpr(std::is_same<launch_arg_t, empty_t>::value &&
    std::is_same<comp_t, less_t<int> >::value &&
    launcher_points_to_t<needles_it, int>::value &&
    launcher_points_to_t<haystack_it, int>::value &&
    launcher_points_to_t<indices_it, int, true>::value) {
    size_t bytes = mgpu_hip_sorted_search_workspace_bytes(num_needles,
      num_haystack);
    mem_t<char> workspace(bytes, context);
    launcher_check(mgpu_hip_sorted_search(needles, num_needles, haystack,
      num_haystack, upper ? MGPU_BOUNDS_UPPER : MGPU_BOUNDS_LOWER, indices,
      workspace.data(), bytes, context.stream()));
    launcher_count_call();
    return true;
  } else
    return false;
}

// inner_join of int keys ordered by less_t<int>: both steps of the layer,
// with the count taken back in between as the header-only path does.
template<typename launch_arg_t, typename a_it, typename b_it, typename comp_t>
bool launcher_inner_join(a_it a, int a_count, b_it b, int b_count, comp_t,
  context_t& context, mem_t<int2>& output) {
  if constexpr(std::is_same<launch_arg_t, empty_t>::value &&
    std::is_same<comp_t, less_t<int> >::value &&
    launcher_points_to_t<a_it, int>::value &&
    launcher_points_to_t<b_it, int>::value) {
    size_t bytes = mgpu_hip_inner_join_workspace_bytes(a_count, b_count);
    mem_t<char> workspace(bytes, context);
    // The count goes to a word of pinned host memory, which holds it as soon
    // as the kernel that stores it has ended: the host looks at the word for
    // a while (the kernels behind that one may still run) before it falls
    // back on waiting for the whole stream.
    mem_t<int> total(1, context, memory_space_host);
    volatile int* word = total.data();
    *word = -1;
    launcher_check(mgpu_hip_inner_join_count(a, a_count, b, b_count,
      total.data(), workspace.data(), bytes, context.stream()));
    for(long spins = 0; *word < 0 && spins < 2000000; ++spins) { }
    if(*word < 0) {
      context.synchronize();
      if(*word < 0) throw cuda_exception_t(hipErrorUnknown);
    }
    int join_count = *word;
    output = mem_t<int2>(join_count, context);
    size_t pairs_bytes = mgpu_hip_inner_join_pairs_workspace_bytes(a_count,
      join_count);
    mem_t<char> pairs_workspace(pairs_bytes, context);
    launcher_check(mgpu_hip_inner_join_pairs(a_count, b_count, join_count,
      workspace.data(), (int*)output.data(), pairs_workspace.data(),
      pairs_bytes, context.stream()));
    launcher_count_call();
    return true;
  } else
    return false;
}

// load_balance_partitions into an int array.
template<typename segments_it>
bool launcher_load_balance_partitions(int64_t count, segments_it segments,
  int num_segments, int spacing, int* partitions, context_t& context) {
  if constexpr(launcher_points_to_t<segments_it, int>::value) {
    launcher_check(mgpu_hip_load_balance_partitions(count, segments,
      num_segments, spacing, partitions, context.stream()));
    launcher_count_call();
    return true;
  } else
    return false;
}

#else // !MGPU_HIP_LAUNCHER

template<typename launch_arg_t, typename... args_t>
constexpr bool launcher_segreduce(const args_t&...) { return false; }
template<typename launch_arg_t, typename... args_t>
constexpr bool launcher_spmv(const args_t&...) { return false; }
template<typename launch_arg_t, typename... args_t>
constexpr bool launcher_load_balance_search(const args_t&...) {
  return false;
}
template<typename launch_arg_t, typename... args_t>
constexpr bool launcher_interval(const args_t&...) { return false; }
template<typename launch_arg_t, typename... args_t>
constexpr bool launcher_scan(const args_t&...) { return false; }
template<typename launch_arg_t, typename... args_t>
constexpr bool launcher_reduce(const args_t&...) { return false; }
template<typename launch_arg_t, typename... args_t>
constexpr bool launcher_sorted_search(const args_t&...) { return false; }
template<typename launch_arg_t, typename... args_t>
constexpr bool launcher_inner_join(const args_t&...) { return false; }
template<typename... args_t>
constexpr bool launcher_load_balance_partitions(const args_t&...) {
  return false;
}

#endif

} // namespace detail

END_MGPU_NAMESPACE
