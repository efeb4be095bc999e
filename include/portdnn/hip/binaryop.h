// sycldnn::binaryop on the HIP backend
// (include/portdnn/binaryop/{operators,params,launch}.h).
#ifndef PORTDNN_HIP_BINARYOP_H_
#define PORTDNN_HIP_BINARYOP_H_

#include <type_traits>
#include <vector>

#include "portdnn/hip/core.h"
#include "snn_hip.h"

namespace sycldnn {
namespace binaryop {

// binaryop/params.h:32.
static constexpr int MAX_DIMS = 4;

// Field for field the reference's record (binaryop/params.h:35-46).
struct BinaryParams {
  using Index = int;
  std::vector<Index> lhs_dims;
  std::vector<Index> rhs_dims;
};

// binaryop/operators.h:27-33.
struct Add {};
struct Sub {};
struct Mul {};
struct Div {};

namespace internal {
template <typename Op>
struct OpCode;
template <>
struct OpCode<Add> {
  static constexpr int value = SNN_HIP_BINARY_ADD;
};
template <>
struct OpCode<Sub> {
  static constexpr int value = SNN_HIP_BINARY_SUB;
};
template <>
struct OpCode<Mul> {
  static constexpr int value = SNN_HIP_BINARY_MUL;
};
template <>
struct OpCode<Div> {
  static constexpr int value = SNN_HIP_BINARY_DIV;
};
}  // namespace internal

// out = lhs Op rhs with the operands broadcast against each other
// (binaryop/launch.h:61-85): dimensions right-aligned, at most MAX_DIMS each
// (none = scalar), a dimension of 1 repeats.  Shapes that do not broadcast
// or have more than MAX_DIMS dimensions give InvalidParameter
// (internal/binaryop/launch.h:40-62, :84-89).
template <typename T, typename Op, typename Backend>
SNNStatus launch(typename Backend::template pointer_type<T const> lhs,
                 typename Backend::template pointer_type<T const> rhs,
                 typename Backend::template pointer_type<T> out,
                 const BinaryParams& params, Backend& backend,
                 const std::vector<hip::Event>& events = {}) {
  hipStream_t stream = backend.get_stream();
  hip::detail::wait_for(stream, events);
  constexpr int op = internal::OpCode<Op>::value;
  const int n_lhs = static_cast<int>(params.lhs_dims.size());
  const int n_rhs = static_cast<int>(params.rhs_dims.size());
  int code;
  if (std::is_same<T, float>::value) {
    code = snn_hip_binaryop_f32(
        reinterpret_cast<const float*>(lhs), reinterpret_cast<const float*>(rhs),
        reinterpret_cast<float*>(out), params.lhs_dims.data(), n_lhs,
        params.rhs_dims.data(), n_rhs, op, stream);
  } else {
    static_assert(std::is_same<T, float>::value || sizeof(T) == 2,
                  "supported data types: float and half");
    code = snn_hip_binaryop_f16(lhs, rhs, out, params.lhs_dims.data(), n_lhs,
                                params.rhs_dims.data(), n_rhs, op, stream);
  }
  return hip::detail::finish(code, stream);
}

}  // namespace binaryop
}  // namespace sycldnn

#endif  // PORTDNN_HIP_BINARYOP_H_
