// libmgpu_hip: segreduce kernels for uint32_t.
#include "segreduce_impl.hxx"
namespace mgpu_hip {
template int segreduce_typed<uint32_t>(const uint32_t*, int, const int*, int, uint32_t*, int,
  uint32_t, void*, void*, int);
}
