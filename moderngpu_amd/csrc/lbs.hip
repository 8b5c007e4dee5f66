// libmgpu_hip: extern "C" entry points of the load-balancing search family.
// Declarations and the reference citations are in include/mgpu_hip.h.
#include "launcher_common.hxx"

using namespace mgpu;
using namespace mgpu_hip;

namespace {

// Tiles of the kernels with cached values (expand, gather, scatter, move);
// the workspace is sized for these, the smaller ones.  Kernels without cached
// values (the search itself) use larger tiles and so fewer splits.
typedef detail::lbs_launch_default_t lbs_launch_t;
typedef detail::lbs_launch_plain_t lbs_plain_launch_t;
static_assert(lbs_plain_launch_t::sm_ptx::nt * lbs_plain_launch_t::sm_ptx::vt >=
  lbs_launch_t::sm_ptx::nt * lbs_launch_t::sm_ptx::vt,
  "the workspace is sized for the smaller tile");

// Plain byte bags for bit-for-bit element copies.
struct alignas(16) bytes16_t { uint64_t lo, hi; };
template<int bytes> struct bytes_type_t;
template<> struct bytes_type_t<1> { typedef uint8_t type; };
template<> struct bytes_type_t<2> { typedef uint16_t type; };
template<> struct bytes_type_t<4> { typedef uint32_t type; };
template<> struct bytes_type_t<8> { typedef uint64_t type; };
template<> struct bytes_type_t<16> { typedef bytes16_t type; };

size_t partition_ints(int count, int num_segments) {
  return detail::lbs_partition_ints(count + num_segments,
    lbs_launch_t::sm_ptx::nt * lbs_launch_t::sm_ptx::vt);
}

bool lbs_args_ok(int count, const int* segments, int num_segments,
  void* workspace, size_t workspace_bytes) {
  if(!sizes_ok(count, num_segments) || (num_segments && !segments))
    return false;
  size_t need = mgpu_hip_lbs_workspace_bytes(count, num_segments);
  return !need || (workspace && workspace_bytes >= need);
}

struct store_seg_rank_f {
  int* seg_out; int* rank_out;
  MGPU_DEVICE void operator()(int index, int seg, int rank, tuple<>) const {
    if(seg_out) seg_out[index] = seg;
    if(rank_out) rank_out[index] = rank;
  }
};

typedef detail::lbs_store_seg_f<int*> store_seg_f;

template<typename type_t>
using expand_f = detail::interval_expand_f<type_t, type_t*>;
// gather / scatter / move: the library's own pointer functors (W consecutive
// items per call for elements of less than 16 bytes).
template<typename type_t>
using gather_f = typename detail::interval_copy_select_t<false, true,
  const type_t*, type_t*>::type;
template<typename type_t>
using scatter_f = typename detail::interval_copy_select_t<true, false,
  const type_t*, type_t*>::type;
template<typename type_t>
using move_f = typename detail::interval_copy_select_t<true, true,
  const type_t*, type_t*>::type;

template<int bytes>
int expand_sized(const void* input, int count, const int* segments,
  int num_segments, void* output, void* workspace, void* stream, int phases) {
  typedef typename bytes_type_t<bytes>::type type_t;
  return guarded(stream, [&](context_t& context) {
    detail::transform_lbs_launch<lbs_launch_t>(
      expand_f<type_t> { (type_t*)output }, count, segments, num_segments,
      make_tuple((const type_t*)input), (int*)workspace, phases, context);
  });
}
template<int bytes>
int gather_sized(const void* input, int count, const int* segments,
  int num_segments, const int* gather, void* output, void* workspace,
  void* stream) {
  typedef typename bytes_type_t<bytes>::type type_t;
  return guarded(stream, [&](context_t& context) {
    detail::transform_lbs_launch<lbs_launch_t>(
      gather_f<type_t> { (const type_t*)input, (type_t*)output }, count,
      segments, num_segments, make_tuple(gather), (int*)workspace,
      detail::lbs_phase_all, context);
  });
}
template<int bytes>
int scatter_sized(const void* input, int count, const int* segments,
  int num_segments, const int* scatter, void* output, void* workspace,
  void* stream) {
  typedef typename bytes_type_t<bytes>::type type_t;
  return guarded(stream, [&](context_t& context) {
    detail::transform_lbs_launch<lbs_launch_t>(
      scatter_f<type_t> { (const type_t*)input, (type_t*)output }, count,
      segments, num_segments, make_tuple(scatter), (int*)workspace,
      detail::lbs_phase_all, context);
  });
}
template<int bytes>
int move_sized(const void* input, int count, const int* segments,
  int num_segments, const int* scatter, const int* gather, void* output,
  void* workspace, void* stream) {
  typedef typename bytes_type_t<bytes>::type type_t;
  return guarded(stream, [&](context_t& context) {
    detail::transform_lbs_launch<lbs_launch_t>(
      move_f<type_t> { (const type_t*)input, (type_t*)output }, count,
      segments, num_segments, make_tuple(scatter, gather), (int*)workspace,
      detail::lbs_phase_all, context);
  });
}

#define MGPU_BY_ELEM_BYTES(fn, ...)                                          \
  switch(elem_bytes) {                                                        \
    case 1: return fn<1>(__VA_ARGS__);                                        \
    case 2: return fn<2>(__VA_ARGS__);                                        \
    case 4: return fn<4>(__VA_ARGS__);                                        \
    case 8: return fn<8>(__VA_ARGS__);                                        \
    case 16: return fn<16>(__VA_ARGS__);                                      \
  }                                                                           \
  return (int)hipErrorInvalidValue;

} // namespace

extern "C" {

size_t mgpu_hip_lbs_workspace_bytes(int count, int num_segments) {
  if(!sizes_ok(count, num_segments)) return 0;
  if(!(count + num_segments)) return 0;
  return sizeof(int) * partition_ints(count, num_segments);
}

int mgpu_hip_load_balance_search_phases(int count, const int* segments,
  int num_segments, int* output, void* workspace, size_t workspace_bytes,
  mgpu_stream_t stream, int phases) {
  if(!lbs_args_ok(count, segments, num_segments, workspace, workspace_bytes) ||
    (count && !output))
    return (int)hipErrorInvalidValue;
  return guarded(stream, [&](context_t& context) {
    detail::transform_lbs_launch<lbs_plain_launch_t>(store_seg_f { output },
      count, segments, num_segments, tuple<>(), (int*)workspace, phases,
      context);
  });
}

int mgpu_hip_load_balance_search(int count, const int* segments,
  int num_segments, int* output, void* workspace, size_t workspace_bytes,
  mgpu_stream_t stream) {
  return mgpu_hip_load_balance_search_phases(count, segments, num_segments,
    output, workspace, workspace_bytes, stream, detail::lbs_phase_all);
}

int mgpu_hip_transform_lbs(int count, const int* segments, int num_segments,
  int* seg_out, int* rank_out, void* workspace, size_t workspace_bytes,
  mgpu_stream_t stream) {
  if(!lbs_args_ok(count, segments, num_segments, workspace, workspace_bytes))
    return (int)hipErrorInvalidValue;
  return guarded(stream, [&](context_t& context) {
    detail::transform_lbs_launch<lbs_plain_launch_t>(
      store_seg_rank_f { seg_out, rank_out }, count, segments, num_segments,
      tuple<>(), (int*)workspace, detail::lbs_phase_all, context);
  });
}

int mgpu_hip_interval_expand_phases(const void* input, int elem_bytes,
  int count, const int* segments, int num_segments, void* output,
  void* workspace, size_t workspace_bytes, mgpu_stream_t stream, int phases) {
  if(!lbs_args_ok(count, segments, num_segments, workspace, workspace_bytes) ||
    (count && (!output || !input)))
    return (int)hipErrorInvalidValue;
  MGPU_BY_ELEM_BYTES(expand_sized, input, count, segments, num_segments,
    output, workspace, stream, phases)
}

int mgpu_hip_interval_expand(const void* input, int elem_bytes, int count,
  const int* segments, int num_segments, void* output, void* workspace,
  size_t workspace_bytes, mgpu_stream_t stream) {
  return mgpu_hip_interval_expand_phases(input, elem_bytes, count, segments,
    num_segments, output, workspace, workspace_bytes, stream,
    detail::lbs_phase_all);
}

int mgpu_hip_interval_gather(const void* input, int elem_bytes, int count,
  const int* segments, int num_segments, const int* gather, void* output,
  void* workspace, size_t workspace_bytes, mgpu_stream_t stream) {
  if(!lbs_args_ok(count, segments, num_segments, workspace, workspace_bytes) ||
    (count && (!output || !input || !gather)))
    return (int)hipErrorInvalidValue;
  MGPU_BY_ELEM_BYTES(gather_sized, input, count, segments, num_segments,
    gather, output, workspace, stream)
}

int mgpu_hip_interval_scatter(const void* input, int elem_bytes, int count,
  const int* segments, int num_segments, const int* scatter, void* output,
  void* workspace, size_t workspace_bytes, mgpu_stream_t stream) {
  if(!lbs_args_ok(count, segments, num_segments, workspace, workspace_bytes) ||
    (count && (!output || !input || !scatter)))
    return (int)hipErrorInvalidValue;
  MGPU_BY_ELEM_BYTES(scatter_sized, input, count, segments, num_segments,
    scatter, output, workspace, stream)
}

int mgpu_hip_interval_move(const void* input, int elem_bytes, int count,
  const int* segments, int num_segments, const int* scatter,
  const int* gather, void* output, void* workspace, size_t workspace_bytes,
  mgpu_stream_t stream) {
  if(!lbs_args_ok(count, segments, num_segments, workspace, workspace_bytes) ||
    (count && (!output || !input || !scatter || !gather)))
    return (int)hipErrorInvalidValue;
  MGPU_BY_ELEM_BYTES(move_sized, input, count, segments, num_segments,
    scatter, gather, output, workspace, stream)
}

} // extern "C"
