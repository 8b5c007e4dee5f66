// libmgpu_hip: segreduce kernels for float.
#include "segreduce_impl.hxx"
namespace mgpu_hip {
template int segreduce_typed<float>(const float*, int, const int*, int, float*, int,
  float, void*, void*, int);
}
