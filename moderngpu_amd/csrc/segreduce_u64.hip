// libmgpu_hip: segreduce kernels for uint64_t.
#include "segreduce_impl.hxx"
namespace mgpu_hip {
template int segreduce_typed<uint64_t>(const uint64_t*, int, const int*, int, uint64_t*, int,
  uint64_t, void*, void*, int);
}
