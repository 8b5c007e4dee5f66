// libmgpu_hip: segreduce kernels for int32_t.
#include "segreduce_impl.hxx"
namespace mgpu_hip {
template int segreduce_typed<int32_t>(const int32_t*, int, const int*, int, int32_t*, int,
  int32_t, void*, void*, int);
}
