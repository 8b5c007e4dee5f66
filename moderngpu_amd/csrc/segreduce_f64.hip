// libmgpu_hip: segreduce kernels for double.
#include "segreduce_impl.hxx"
namespace mgpu_hip {
template int segreduce_typed<double>(const double*, int, const int*, int, double*, int,
  double, void*, void*, int);
}
