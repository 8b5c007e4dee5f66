// Shared pieces of the extern "C" launcher layer (libmgpu_hip.so).
#pragma once
#include <moderngpu/kernel_segreduce.hxx>
#include <moderngpu/kernel_load_balance.hxx>
#include <moderngpu/kernel_intervalmove.hxx>
#include "../../include/mgpu_hip.h"

namespace mgpu_hip {

// A context that only carries the caller's stream.  The launcher layer never
// allocates: asking this context for memory is a programming error.
class stream_context_t : public mgpu::context_t {
  hipStream_t _stream;
  hipDeviceProp_t _props;
public:
  explicit stream_context_t(void* stream) : _stream((hipStream_t)stream) {
    memset(&_props, 0, sizeof(_props));
  }
  virtual const hipDeviceProp_t& props() const { return _props; }
  virtual int ptx_version() const { return mgpu::arch_version_gfx950; }
  virtual hipStream_t stream() { return _stream; }
  virtual void* alloc(size_t, mgpu::memory_space_t) {
    throw mgpu::cuda_exception_t(hipErrorNotSupported);
  }
  virtual void free(void*, mgpu::memory_space_t) { }
  virtual void synchronize() { }
  virtual hipEvent_t event() { return nullptr; }
  virtual void timer_begin() { }
  virtual double timer_end() { return 0; }
};

// Runs body(context), mapping exceptions to return codes.
template<typename body_t>
int guarded(void* stream, body_t body) {
  try {
    stream_context_t context(stream);
    body(context);
    return (int)hipSuccess;
  } catch(const mgpu::cuda_exception_t& e) {
    return (int)e.result;
  } catch(...) {
    return (int)hipErrorUnknown;
  }
}

// Argument checks common to every entry point: sizes fit the 32-bit index
// space and non-empty arrays have pointers.
inline bool sizes_ok(int count, int num_segments) {
  return count >= 0 && num_segments >= 0 &&
    (int64_t)count + num_segments < ((int64_t)1 << 31);
}

inline size_t value_size(int dtype) {
  switch(dtype) {
    case MGPU_I32: case MGPU_U32: case MGPU_F32: return 4;
    case MGPU_I64: case MGPU_U64: case MGPU_F64: return 8;
  }
  return 0;
}

template<typename type_t>
struct segreduce_launch_t {
  typedef typename mgpu::detail::segreduce_launch_default_t<type_t>::type_t_
    type;
};

// Typed segreduce over pointers; defined per value type in segreduce_*.hip.
template<typename type_t>
int segreduce_typed(const type_t* input, int count, const int* segments,
  int num_segments, type_t* output, int op, type_t init, void* workspace,
  void* stream, int phases);

} // namespace mgpu_hip
