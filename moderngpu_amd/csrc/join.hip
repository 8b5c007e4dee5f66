// libmgpu_hip: sorted_search and inner_join for int keys ordered by less_t.
#include "launcher_common.hxx"
#include <moderngpu/kernel_join.hxx>

using namespace mgpu;
using namespace mgpu_hip;

namespace {

typedef detail::sorted_search_launch_default_t search_launch_t;
typedef detail::lbs_launch_default_t lbs_launch_t;
typedef detail::scan_launch_default_t<int>::type_t_ scan_launch_t;

int search_nv() {
  return search_launch_t::sm_ptx::nt * search_launch_t::sm_ptx::vt;
}
size_t search_partitions(int num_needles, int num_haystack) {
  return (size_t)div_up((int64_t)num_needles + num_haystack,
    (int64_t)search_nv()) + 1;
}
size_t search_samples(int num_needles, int num_haystack) {
  return detail::sorted_search_sample_count(num_needles, num_haystack,
    search_nv());
}
// The splits, then (256-byte aligned) the key samples.
size_t search_samples_offset(int num_needles, int num_haystack) {
  return (sizeof(int) * search_partitions(num_needles, num_haystack) + 255) &
    ~(size_t)255;
}

// Temporaries of mgpu_hip_inner_join_count, which mgpu_hip_inner_join_pairs
// reads again.
struct join_workspace_t {
  int* lower; int* matches; int* starts; int* partitions; int* samples;
  int* partials;
  size_t bytes;
  join_workspace_t(int a_count, int b_count, void* base) {
    char* at = (char*)base;
    auto take = [&](size_t ints) {
      int* p = (int*)at;
      at += (sizeof(int) * ints + 255) & ~(size_t)255;
      return p;
    };
    lower = take(a_count);
    matches = take(a_count);
    starts = take(a_count);
    partitions = take(search_partitions(a_count, b_count));
    samples = take(search_samples(a_count, b_count));
    partials = take(detail::scan_partials_count(a_count,
      scan_launch_t::sm_ptx::nt * scan_launch_t::sm_ptx::vt));
    bytes = (size_t)(at - (char*)base);
  }
};

bool keys_ok(const int* a, int a_count, const int* b, int b_count) {
  return sizes_ok(a_count, b_count) && (!a_count || a) && (!b_count || b);
}

} // namespace

extern "C" {

size_t mgpu_hip_sorted_search_workspace_bytes(int num_needles,
  int num_haystack) {
  if(!sizes_ok(num_needles, num_haystack)) return 0;
  return search_samples_offset(num_needles, num_haystack) +
    sizeof(int) * search_samples(num_needles, num_haystack);
}

int mgpu_hip_sorted_search(const int* needles, int num_needles,
  const int* haystack, int num_haystack, int bounds, int* indices,
  void* workspace, size_t workspace_bytes, mgpu_stream_t stream) {
  if(!keys_ok(needles, num_needles, haystack, num_haystack) ||
    (num_needles && !indices) ||
    (bounds != MGPU_BOUNDS_LOWER && bounds != MGPU_BOUNDS_UPPER))
    return (int)hipErrorInvalidValue;
  if(!num_needles) return (int)hipSuccess;
  if(!workspace || workspace_bytes <
    mgpu_hip_sorted_search_workspace_bytes(num_needles, num_haystack))
    return (int)hipErrorInvalidValue;
  int* samples = (int*)((char*)workspace +
    search_samples_offset(num_needles, num_haystack));
  return guarded(stream, [&](context_t& context) {
    if(MGPU_BOUNDS_LOWER == bounds)
      detail::sorted_search_launch<bounds_lower, search_launch_t>(needles,
        num_needles, haystack, num_haystack, indices, less_t<int>(),
        (int*)workspace, samples, context);
    else
      detail::sorted_search_launch<bounds_upper, search_launch_t>(needles,
        num_needles, haystack, num_haystack, indices, less_t<int>(),
        (int*)workspace, samples, context);
  });
}

size_t mgpu_hip_inner_join_workspace_bytes(int a_count, int b_count) {
  if(!sizes_ok(a_count, b_count)) return 0;
  return join_workspace_t(a_count, b_count, nullptr).bytes;
}

int mgpu_hip_inner_join_count(const int* a, int a_count, const int* b,
  int b_count, int* join_count, void* workspace, size_t workspace_bytes,
  mgpu_stream_t stream) {
  if(!keys_ok(a, a_count, b, b_count) || !join_count)
    return (int)hipErrorInvalidValue;
  join_workspace_t ws(a_count, b_count, workspace);
  if(ws.bytes && (!workspace || workspace_bytes < ws.bytes))
    return (int)hipErrorInvalidValue;
  return guarded(stream, [&](context_t& context) {
    // One search: the lower bound of every a key and the number of b keys
    // equal to it; then the scan of those numbers.
    detail::join_count_launch<search_launch_t>(a, a_count, b, b_count,
      less_t<int>(), ws.lower, ws.matches, ws.starts, ws.partitions,
      ws.samples, ws.partials, join_count, context);
  });
}

size_t mgpu_hip_inner_join_pairs_workspace_bytes(int a_count,
  int64_t join_count) {
  if(a_count < 0 || join_count < 0 ||
    join_count + a_count >= ((int64_t)1 << 31))
    return 0;
  return sizeof(int) * detail::lbs_partition_ints((int)join_count + a_count,
    lbs_launch_t::sm_ptx::nt * lbs_launch_t::sm_ptx::vt);
}

int mgpu_hip_inner_join_pairs(int a_count, int b_count, int join_count,
  const void* count_workspace, int* pairs, void* workspace,
  size_t workspace_bytes, mgpu_stream_t stream) {
  if(!sizes_ok(a_count, b_count) || !sizes_ok(join_count, a_count) ||
    (join_count && (!pairs || !count_workspace)))
    return (int)hipErrorInvalidValue;
  if(!join_count) return (int)hipSuccess;
  size_t need = mgpu_hip_inner_join_pairs_workspace_bytes(a_count,
    join_count);
  if(!workspace || workspace_bytes < need) return (int)hipErrorInvalidValue;
  join_workspace_t ws(a_count, b_count, (void*)count_workspace);
  return guarded(stream, [&](context_t& context) {
    detail::transform_lbs_launch<lbs_launch_t>(
      detail::join_pairs_f { (int2*)pairs }, join_count,
      (const int*)ws.starts, a_count, make_tuple((const int*)ws.lower),
      (int*)workspace, detail::lbs_phase_all, context);
  });
}

} // extern "C"
