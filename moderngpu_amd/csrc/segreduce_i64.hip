// libmgpu_hip: segreduce kernels for int64_t.
#include "segreduce_impl.hxx"
namespace mgpu_hip {
template int segreduce_typed<int64_t>(const int64_t*, int, const int*, int, int64_t*, int,
  int64_t, void*, void*, int);
}
