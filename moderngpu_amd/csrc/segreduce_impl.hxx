// Instantiates segreduce for one value type and the three built-in operators.
#pragma once
#include "launcher_common.hxx"

namespace mgpu_hip {

template<typename type_t>
int segreduce_typed(const type_t* input, int count, const int* segments,
  int num_segments, type_t* output, int op, type_t init, void* workspace,
  void* stream, int phases) {
  using namespace mgpu;
  typedef typename segreduce_launch_t<type_t>::type launch_t;
  return guarded(stream, [&](context_t& context) {
    detail::segreduce_workspace_t ws(count, num_segments,
      launch_t::nv(context), sizeof(type_t));
    switch(op) {
      case MGPU_PLUS:
        detail::segreduce_launch<launch_t>(input, count, segments,
          num_segments, output, plus_t<type_t>(), init, workspace, ws,
          context, phases);
        break;
      case MGPU_MAXIMUM:
        detail::segreduce_launch<launch_t>(input, count, segments,
          num_segments, output, maximum_t<type_t>(), init, workspace, ws,
          context, phases);
        break;
      case MGPU_MINIMUM:
        detail::segreduce_launch<launch_t>(input, count, segments,
          num_segments, output, minimum_t<type_t>(), init, workspace, ws,
          context, phases);
        break;
      default:
        throw cuda_exception_t(hipErrorInvalidValue);
    }
  });
}

} // namespace mgpu_hip
