// sycldnn::matmul on the HIP backend
// (include/portdnn/matmul/{params,launch}.h).
#ifndef PORTDNN_HIP_MATMUL_H_
#define PORTDNN_HIP_MATMUL_H_

#include <type_traits>
#include <vector>

#include "portdnn/hip/core.h"
#include "snn_hip.h"

namespace sycldnn {
namespace matmul {

// Field for field the reference's record (matmul/params.h:29-55).
struct MatmulParams {
  using Index = int;
  Index batches;
  Index m;
  Index k;
  Index n;
  float beta;
  sycldnn::BatchFormat batch_type = sycldnn::BatchFormat::STRIDED;
};

// output[i] = beta * output[i] + op(lhs[i]) * op(rhs[i]) for every batch i,
// row-major, op(X) = X^T when TransposeX (matmul/launch.h:80-90).  Sizes
// that are not positive give InvalidParameter as in
// internal/matmul/launch.h:66-70; interleaved batches are not implemented
// (the reference's backends reject them too,
// snn_usm_matmul_provider.h:217-220) and give InvalidAlgorithm.
template <typename T, bool TransposeLHS, bool TransposeRHS, typename Backend>
SNNStatus launch(typename Backend::template pointer_type<T const> lhs,
                 typename Backend::template pointer_type<T const> rhs,
                 typename Backend::template pointer_type<T> output,
                 MatmulParams const& params, Backend& backend,
                 const std::vector<hip::Event>& events = {}) {
  hipStream_t stream = backend.get_stream();
  if (params.batch_type != sycldnn::BatchFormat::STRIDED)
    return hip::detail::finish(SNN_HIP_INVALID_ALGORITHM, stream);
  hip::detail::wait_for(stream, events);
  int code;
  if constexpr (std::is_same<T, float>::value) {
    code = snn_hip_matmul_f32(lhs, rhs, output, params.batches, params.m,
                              params.k, params.n, TransposeLHS, TransposeRHS,
                              params.beta, stream);
  } else {
    static_assert(sizeof(T) == 2, "supported data types: float and half");
    code = snn_hip_matmul_f16(lhs, rhs, output, params.batches, params.m,
                              params.k, params.n, TransposeLHS, TransposeRHS,
                              params.beta, stream);
  }
  return hip::detail::finish(code, stream);
}

}  // namespace matmul
}  // namespace sycldnn

#endif  // PORTDNN_HIP_MATMUL_H_
