// libmgpu_hip: extern "C" entry points for partitioning, segreduce dispatch
// and spmv.  Declarations and the reference citations are in
// include/mgpu_hip.h.
#include "launcher_common.hxx"
#include <atomic>

using namespace mgpu;
using namespace mgpu_hip;

// Device memory of mgpu_hip_segreduce_static: what mgpu_hip_segreduce takes
// as its workspace argument (tile splits and one carry per tile), held by the
// library itself so that the call allocates nothing.  Every GPU the library
// runs on has its own copy at its own address; host code may only use the
// address hipGetSymbolAddress returns, never the symbol's name.
static __device__ __align__(256) unsigned char scratch[MGPU_HIP_STATIC_SCRATCH_BYTES];

namespace {

// Address of `scratch` on the current device, looked up once per device.
enum { max_scratch_devices = 64 };
std::atomic<void*> scratch_address[max_scratch_devices];

int static_scratch(void** address) {
  int device = -1;
  hipError_t result = hipGetDevice(&device);
  if(hipSuccess != result) return (int)result;
  if(device < 0 || device >= max_scratch_devices)
    return (int)hipErrorInvalidDevice;
  void* p = scratch_address[device].load(std::memory_order_acquire);
  if(!p) {
    result = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if(hipSuccess != result) return (int)result;
    if(!p) return (int)hipErrorInvalidSymbol;
    scratch_address[device].store(p, std::memory_order_release);
  }
  *address = p;
  return (int)hipSuccess;
}

template<typename type_t>
int segreduce_any(const void* input, int count, const int* segments,
  int num_segments, void* output, int op, const void* init, void* workspace,
  void* stream, int phases) {
  return segreduce_typed<type_t>((const type_t*)input, count, segments,
    num_segments, (type_t*)output, op, *(const type_t*)init, workspace,
    stream, phases);
}

template<typename type_t>
int spmv_typed(const type_t* matrix, const int* columns, const type_t* vector,
  int count, const int* segments, int num_segments, type_t* output,
  void* workspace, void* stream, int phases) {
  typedef typename segreduce_launch_t<type_t>::type launch_t;
  return guarded(stream, [&](context_t& context) {
    detail::segreduce_workspace_t ws(count, num_segments,
      launch_t::nv(context), sizeof(type_t));
    detail::segreduce_launch<launch_t>(
      detail::spmv_input_t<type_t> { matrix, columns, vector }, count,
      segments, num_segments, output, plus_t<type_t>(), (type_t)0, workspace,
      ws, context, phases);
  });
}

struct seg_plus_rank_f {
  MGPU_DEVICE int operator()(int, int seg, int rank, tuple<>) const {
    return seg + rank;
  }
};
struct mod13_f {
  MGPU_DEVICE int operator()(int index) const { return index % 13; }
};

} // namespace

extern "C" {

int mgpu_hip_version(void) { return 10000; }

const char* mgpu_hip_error_string(int code) {
  return hipGetErrorString((hipError_t)code);
}

int mgpu_hip_memory_properties(int device, int* clock_khz,
  int* bus_width_bits) {
  if(!clock_khz || !bus_width_bits) return (int)hipErrorInvalidValue;
  hipDeviceProp_t prop;
  hipError_t result = hipGetDeviceProperties(&prop, device);
  if(hipSuccess != result) return (int)result;
  *clock_khz = prop.memoryClockRate;
  *bus_width_bits = prop.memoryBusWidth;
  return 0;
}

int mgpu_hip_segreduce_tile_size(int dtype) {
  switch(value_size(dtype)) {
    case 4: return segreduce_launch_t<float>::type::sm_ptx::nt *
      segreduce_launch_t<float>::type::sm_ptx::vt;
    case 8: return segreduce_launch_t<double>::type::sm_ptx::nt *
      segreduce_launch_t<double>::type::sm_ptx::vt;
  }
  return 0;
}

int mgpu_hip_lbs_tile_size(void) {
  return detail::lbs_tile_spacing(detail::lbs_launch_default_t::sm_ptx::nt *
    detail::lbs_launch_default_t::sm_ptx::vt);
}

int mgpu_hip_lbs_search_tile_size(void) {
  return detail::lbs_tile_spacing(detail::lbs_launch_plain_t::sm_ptx::nt *
    detail::lbs_launch_plain_t::sm_ptx::vt);
}

int mgpu_hip_partition_count(int64_t a_count, int64_t b_count,
  int64_t spacing) {
  if(a_count < 0 || b_count < 0 || spacing <= 0) return 0;
  return (int)div_up(a_count + b_count, spacing) + 1;
}

int mgpu_hip_load_balance_partitions(int64_t count, const int* segments,
  int num_segments, int spacing, int* partitions, mgpu_stream_t stream) {
  if(count < 0 || num_segments < 0 || spacing <= 0 || !partitions ||
    count + num_segments >= ((int64_t)1 << 31) || (num_segments && !segments))
    return (int)hipErrorInvalidValue;
  return guarded(stream, [&](context_t& context) {
    load_balance_partitions_into(count, segments, num_segments, spacing,
      partitions, context);
  });
}

int mgpu_hip_merge_path_partitions(const int* a_keys, int64_t a_count,
  const int* b_keys, int64_t b_count, int64_t spacing, int bounds,
  int* partitions, mgpu_stream_t stream) {
  if(a_count < 0 || b_count < 0 || spacing <= 0 || !partitions ||
    a_count + b_count >= ((int64_t)1 << 31) || (b_count && !b_keys) ||
    (bounds != MGPU_BOUNDS_LOWER && bounds != MGPU_BOUNDS_UPPER))
    return (int)hipErrorInvalidValue;
  return guarded(stream, [&](context_t& context) {
    if(a_keys) {
      if(MGPU_BOUNDS_UPPER == bounds)
        merge_path_partitions_into<bounds_upper>(a_keys, a_count, b_keys,
          b_count, spacing, less_t<int>(), partitions, context);
      else
        merge_path_partitions_into<bounds_lower>(a_keys, a_count, b_keys,
          b_count, spacing, less_t<int>(), partitions, context);
    } else {
      counting_iterator_t<int> a(0);
      if(MGPU_BOUNDS_UPPER == bounds)
        merge_path_partitions_into<bounds_upper>(a, a_count, b_keys, b_count,
          spacing, less_t<int>(), partitions, context);
      else
        merge_path_partitions_into<bounds_lower>(a, a_count, b_keys, b_count,
          spacing, less_t<int>(), partitions, context);
    }
  });
}

int mgpu_hip_binary_search_partitions(const int* keys, int count,
  int num_items, int spacing, int bounds, int* partitions,
  mgpu_stream_t stream) {
  if(count < 0 || num_items < 0 || spacing <= 0 || !partitions ||
    (num_items && !keys) ||
    (bounds != MGPU_BOUNDS_LOWER && bounds != MGPU_BOUNDS_UPPER))
    return (int)hipErrorInvalidValue;
  return guarded(stream, [&](context_t& context) {
    int num_partitions = div_up(count, spacing) + 1;
    bool upper = MGPU_BOUNDS_UPPER == bounds;
    transform<256>([=]MGPU_DEVICE(int index) {
      int key = (int)min((int64_t)spacing * index, (int64_t)count);
      partitions[index] = upper ?
        binary_search<bounds_upper>(keys, num_items, key, less_t<int>()) :
        binary_search<bounds_lower>(keys, num_items, key, less_t<int>());
    }, num_partitions, context);
  });
}

size_t mgpu_hip_segreduce_workspace_bytes(int count, int num_segments,
  int dtype) {
  size_t vs = value_size(dtype);
  if(!vs || !sizes_ok(count, num_segments)) return 0;
  detail::segreduce_workspace_t ws(count, num_segments,
    mgpu_hip_segreduce_tile_size(dtype), vs);
  return ws.bytes;
}

int mgpu_hip_segreduce_phases(const void* input, int count,
  const int* segments, int num_segments, void* output, int dtype, int op,
  const void* init, void* workspace, size_t workspace_bytes,
  mgpu_stream_t stream, int phases) {
  if(!sizes_ok(count, num_segments) || !value_size(dtype) || !init ||
    op < MGPU_PLUS || op > MGPU_MINIMUM || (count && !input) ||
    (num_segments && (!segments || !output)))
    return (int)hipErrorInvalidValue;
  size_t need = mgpu_hip_segreduce_workspace_bytes(count, num_segments, dtype);
  if(need && (!workspace || workspace_bytes < need))
    return (int)hipErrorInvalidValue;

  switch(dtype) {
    case MGPU_I32: return segreduce_any<int32_t>(input, count, segments, num_segments, output, op, init, workspace, stream, phases);
    case MGPU_U32: return segreduce_any<uint32_t>(input, count, segments, num_segments, output, op, init, workspace, stream, phases);
    case MGPU_I64: return segreduce_any<int64_t>(input, count, segments, num_segments, output, op, init, workspace, stream, phases);
    case MGPU_U64: return segreduce_any<uint64_t>(input, count, segments, num_segments, output, op, init, workspace, stream, phases);
    case MGPU_F32: return segreduce_any<float>(input, count, segments, num_segments, output, op, init, workspace, stream, phases);
    case MGPU_F64: return segreduce_any<double>(input, count, segments, num_segments, output, op, init, workspace, stream, phases);
  }
  return (int)hipErrorInvalidValue;
}

int mgpu_hip_segreduce(const void* input, int count, const int* segments,
  int num_segments, void* output, int dtype, int op, const void* init,
  void* workspace, size_t workspace_bytes, mgpu_stream_t stream) {
  return mgpu_hip_segreduce_phases(input, count, segments, num_segments,
    output, dtype, op, init, workspace, workspace_bytes, stream,
    MGPU_PHASE_ALL);
}

int mgpu_hip_segreduce_static(const void* input, int count,
  const int* segments, int num_segments, void* output, int dtype, int op,
  const void* init, mgpu_stream_t stream) {
  if(!sizes_ok(count, num_segments) || !value_size(dtype))
    return (int)hipErrorInvalidValue;
  size_t need = mgpu_hip_segreduce_workspace_bytes(count, num_segments, dtype);
  if(need > (size_t)MGPU_HIP_STATIC_SCRATCH_BYTES)
    return (int)hipErrorOutOfMemory;
  void* workspace = nullptr;
  int result = static_scratch(&workspace);
  if(result) return result;
  // Every piece of the workspace is written by the call before it is read,
  // so what an earlier call left there needs no clearing.
  return mgpu_hip_segreduce_phases(input, count, segments, num_segments,
    output, dtype, op, init, workspace, MGPU_HIP_STATIC_SCRATCH_BYTES, stream,
    MGPU_PHASE_ALL);
}

int mgpu_hip_transform_segreduce_mod13(int count, const int* segments,
  int num_segments, int* output, int init, void* workspace,
  size_t workspace_bytes, mgpu_stream_t stream) {
  if(!sizes_ok(count, num_segments) ||
    (num_segments && (!segments || !output)))
    return (int)hipErrorInvalidValue;
  size_t need = mgpu_hip_segreduce_workspace_bytes(count, num_segments,
    MGPU_I32);
  if(need && (!workspace || workspace_bytes < need))
    return (int)hipErrorInvalidValue;
  typedef segreduce_launch_t<int>::type launch_t;
  return guarded(stream, [&](context_t& context) {
    detail::segreduce_workspace_t ws(count, num_segments,
      launch_t::nv(context), sizeof(int));
    detail::segreduce_launch<launch_t>(make_load_iterator<int>(mod13_f()),
      count, segments, num_segments, output, plus_t<int>(), init, workspace,
      ws, context);
  });
}

int mgpu_hip_lbs_segreduce_seg_plus_rank(int count, const int* segments,
  int num_segments, int* output, int init, void* workspace,
  size_t workspace_bytes, mgpu_stream_t stream) {
  if(!sizes_ok(count, num_segments) ||
    (num_segments && (!segments || !output)))
    return (int)hipErrorInvalidValue;
  size_t need = mgpu_hip_segreduce_workspace_bytes(count, num_segments,
    MGPU_I32);
  if(need && (!workspace || workspace_bytes < need))
    return (int)hipErrorInvalidValue;
  typedef segreduce_launch_t<int>::type launch_t;
  return guarded(stream, [&](context_t& context) {
    detail::segreduce_workspace_t ws(count, num_segments,
      launch_t::nv(context), sizeof(int));
    detail::lbs_input_t<seg_plus_rank_f, tuple<>, int>
      input { seg_plus_rank_f(), tuple<>() };
    detail::segreduce_launch<launch_t>(input, count, segments, num_segments,
      output, plus_t<int>(), init, workspace, ws, context);
  });
}

int mgpu_hip_spmv_phases(const void* matrix, const int* columns,
  const void* vector, int count, const int* segments, int num_segments,
  void* output, int dtype, void* workspace, size_t workspace_bytes,
  mgpu_stream_t stream, int phases) {
  if(!sizes_ok(count, num_segments) ||
    (dtype != MGPU_F32 && dtype != MGPU_F64) ||
    (count && (!matrix || !columns || !vector)) ||
    (num_segments && (!segments || !output)))
    return (int)hipErrorInvalidValue;
  size_t need = mgpu_hip_segreduce_workspace_bytes(count, num_segments, dtype);
  if(need && (!workspace || workspace_bytes < need))
    return (int)hipErrorInvalidValue;
  if(MGPU_F32 == dtype)
    return spmv_typed<float>((const float*)matrix, columns,
      (const float*)vector, count, segments, num_segments, (float*)output,
      workspace, stream, phases);
  return spmv_typed<double>((const double*)matrix, columns,
    (const double*)vector, count, segments, num_segments, (double*)output,
    workspace, stream, phases);
}

int mgpu_hip_spmv(const void* matrix, const int* columns, const void* vector,
  int count, const int* segments, int num_segments, void* output, int dtype,
  void* workspace, size_t workspace_bytes, mgpu_stream_t stream) {
  return mgpu_hip_spmv_phases(matrix, columns, vector, count, segments,
    num_segments, output, dtype, workspace, workspace_bytes, stream,
    MGPU_PHASE_ALL);
}

} // extern "C"
