// libmgpu_hip: device-wide scan and reduce over pointers for the built-in
// value types and operators.
#include "launcher_common.hxx"
#include <moderngpu/kernel_scan.hxx>
#include <moderngpu/kernel_reduce.hxx>

using namespace mgpu;
using namespace mgpu_hip;

namespace {

template<typename type_t>
struct scan_launch_of_t {
  typedef typename detail::scan_launch_default_t<type_t>::type_t_ type;
  static int nv() { return type::sm_ptx::nt * type::sm_ptx::vt; }
};

// A reduction nobody asked for goes to a discard iterator.
template<scan_type_t scan_type, typename type_t, typename op_t>
void scan_one(const type_t* input, int count, type_t* output, op_t op,
  type_t* reduction, void* workspace, context_t& context) {
  typedef typename scan_launch_of_t<type_t>::type launch_t;
  if(reduction)
    detail::scan_launch<scan_type, launch_t>(input, count, output, op,
      reduction, (type_t*)workspace, context);
  else
    detail::scan_launch<scan_type, launch_t>(input, count, output, op,
      discard_iterator_t<type_t>(), (type_t*)workspace, context);
}

template<typename type_t>
int scan_typed(const void* input, int count, void* output, int op,
  int inclusive, void* reduction, void* workspace, void* stream) {
  const type_t* in = (const type_t*)input;
  type_t* out = (type_t*)output;
  type_t* red = (type_t*)reduction;
  return guarded(stream, [&](context_t& context) {
    switch(op) {
      case MGPU_PLUS:
        if(inclusive) scan_one<scan_type_inc>(in, count, out,
          plus_t<type_t>(), red, workspace, context);
        else scan_one<scan_type_exc>(in, count, out, plus_t<type_t>(), red,
          workspace, context);
        break;
      case MGPU_MAXIMUM:
        if(inclusive) scan_one<scan_type_inc>(in, count, out,
          maximum_t<type_t>(), red, workspace, context);
        else scan_one<scan_type_exc>(in, count, out, maximum_t<type_t>(),
          red, workspace, context);
        break;
      case MGPU_MINIMUM:
        if(inclusive) scan_one<scan_type_inc>(in, count, out,
          minimum_t<type_t>(), red, workspace, context);
        else scan_one<scan_type_exc>(in, count, out, minimum_t<type_t>(),
          red, workspace, context);
        break;
      default:
        throw cuda_exception_t(hipErrorInvalidValue);
    }
  });
}

template<typename type_t>
int reduce_typed(const void* input, int count, void* reduction, int op,
  void* workspace, void* stream) {
  typedef typename scan_launch_of_t<type_t>::type launch_t;
  const type_t* in = (const type_t*)input;
  type_t* red = (type_t*)reduction;
  type_t* ws = (type_t*)workspace;
  return guarded(stream, [&](context_t& context) {
    switch(op) {
      case MGPU_PLUS:
        detail::reduce_launch<launch_t>(in, count, red, plus_t<type_t>(), ws,
          context);
        break;
      case MGPU_MAXIMUM:
        detail::reduce_launch<launch_t>(in, count, red, maximum_t<type_t>(),
          ws, context);
        break;
      case MGPU_MINIMUM:
        detail::reduce_launch<launch_t>(in, count, red, minimum_t<type_t>(),
          ws, context);
        break;
      default:
        throw cuda_exception_t(hipErrorInvalidValue);
    }
  });
}

int tile_size(int dtype) {
  switch(dtype) {
    case MGPU_I32: return scan_launch_of_t<int32_t>::nv();
    case MGPU_U32: return scan_launch_of_t<uint32_t>::nv();
    case MGPU_I64: return scan_launch_of_t<int64_t>::nv();
    case MGPU_U64: return scan_launch_of_t<uint64_t>::nv();
    case MGPU_F32: return scan_launch_of_t<float>::nv();
    case MGPU_F64: return scan_launch_of_t<double>::nv();
  }
  return 0;
}

} // namespace

extern "C" {

size_t mgpu_hip_scan_workspace_bytes(int count, int dtype) {
  size_t vs = value_size(dtype);
  if(!vs || count < 0) return 0;
  return vs * detail::scan_partials_count(count, tile_size(dtype));
}

int mgpu_hip_scan(const void* input, int count, void* output, int dtype,
  int op, int inclusive, void* reduction, void* workspace,
  size_t workspace_bytes, mgpu_stream_t stream) {
  if(count < 0 || !value_size(dtype) || op < MGPU_PLUS || op > MGPU_MINIMUM ||
    (count && (!input || !output)))
    return (int)hipErrorInvalidValue;
  size_t need = mgpu_hip_scan_workspace_bytes(count, dtype);
  if(need && (!workspace || workspace_bytes < need))
    return (int)hipErrorInvalidValue;
  switch(dtype) {
    case MGPU_I32: return scan_typed<int32_t>(input, count, output, op, inclusive, reduction, workspace, stream);
    case MGPU_U32: return scan_typed<uint32_t>(input, count, output, op, inclusive, reduction, workspace, stream);
    case MGPU_I64: return scan_typed<int64_t>(input, count, output, op, inclusive, reduction, workspace, stream);
    case MGPU_U64: return scan_typed<uint64_t>(input, count, output, op, inclusive, reduction, workspace, stream);
    case MGPU_F32: return scan_typed<float>(input, count, output, op, inclusive, reduction, workspace, stream);
    case MGPU_F64: return scan_typed<double>(input, count, output, op, inclusive, reduction, workspace, stream);
  }
  return (int)hipErrorInvalidValue;
}

size_t mgpu_hip_reduce_workspace_bytes(int count, int dtype) {
  size_t vs = value_size(dtype);
  if(!vs || count < 0) return 0;
  return vs * detail::reduce_partials_count(count, tile_size(dtype));
}

int mgpu_hip_reduce(const void* input, int count, void* reduction, int dtype,
  int op, void* workspace, size_t workspace_bytes, mgpu_stream_t stream) {
  if(count < 0 || !value_size(dtype) || op < MGPU_PLUS || op > MGPU_MINIMUM ||
    (count && (!input || !reduction)))
    return (int)hipErrorInvalidValue;
  size_t need = mgpu_hip_reduce_workspace_bytes(count, dtype);
  if(need && (!workspace || workspace_bytes < need))
    return (int)hipErrorInvalidValue;
  switch(dtype) {
    case MGPU_I32: return reduce_typed<int32_t>(input, count, reduction, op, workspace, stream);
    case MGPU_U32: return reduce_typed<uint32_t>(input, count, reduction, op, workspace, stream);
    case MGPU_I64: return reduce_typed<int64_t>(input, count, reduction, op, workspace, stream);
    case MGPU_U64: return reduce_typed<uint64_t>(input, count, reduction, op, workspace, stream);
    case MGPU_F32: return reduce_typed<float>(input, count, reduction, op, workspace, stream);
    case MGPU_F64: return reduce_typed<double>(input, count, reduction, op, workspace, stream);
  }
  return (int)hipErrorInvalidValue;
}

} // extern "C"
