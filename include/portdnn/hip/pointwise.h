// sycldnn::pointwise on the HIP backend
// (include/portdnn/pointwise/{operators,direction,launch}.h).
#ifndef PORTDNN_HIP_POINTWISE_H_
#define PORTDNN_HIP_POINTWISE_H_

#include <cstddef>
#include <type_traits>
#include <vector>

#include "portdnn/hip/core.h"
#include "snn_hip.h"

namespace sycldnn {
namespace pointwise {

// pointwise/direction.h:30-34.
struct Forward {};
struct Gradient {};

// pointwise/operators.h:28-44: operator templates over the direction.
template <typename Direction>
struct Relu {};
template <typename Direction>
struct Tanh {};
template <typename Direction>
struct Exp {};
template <typename Direction>
struct Log {};
template <typename Direction>
struct Floor {};
template <typename Direction>
struct Sqrt {};

namespace internal {
template <template <typename> class Op>
struct OpCode;
template <>
struct OpCode<Relu> {
  static constexpr int value = SNN_HIP_POINTWISE_RELU;
};
template <>
struct OpCode<Tanh> {
  static constexpr int value = SNN_HIP_POINTWISE_TANH;
};
template <>
struct OpCode<Exp> {
  static constexpr int value = SNN_HIP_POINTWISE_EXP;
};
template <>
struct OpCode<Log> {
  static constexpr int value = SNN_HIP_POINTWISE_LOG;
};
template <>
struct OpCode<Floor> {
  static constexpr int value = SNN_HIP_POINTWISE_FLOOR;
};
template <>
struct OpCode<Sqrt> {
  static constexpr int value = SNN_HIP_POINTWISE_SQRT;
};
template <typename Direction>
using DisableIfGradient =
    typename std::enable_if<!std::is_same<Direction, Gradient>::value>::type;
template <typename Direction>
using EnableIfGradient =
    typename std::enable_if<std::is_same<Direction, Gradient>::value>::type;
}  // namespace internal

// output[i] = Op(input[i]) (pointwise/launch.h:73-100).  n_items == 0 gives
// InvalidParameter (internal/pointwise/launch_internal.h:69).
template <typename T, template <typename> class PointwiseType,
          typename Direction, typename Backend,
          typename = internal::DisableIfGradient<Direction>>
SNNStatus launch(typename Backend::template pointer_type<T const> input,
                 typename Backend::template pointer_type<T> output,
                 size_t const n_items, Backend& backend,
                 const std::vector<hip::Event>& events = {}) {
  hipStream_t stream = backend.get_stream();
  hip::detail::wait_for(stream, events);
  constexpr int op = internal::OpCode<PointwiseType>::value;
  int code;
  if (std::is_same<T, float>::value) {
    code = snn_hip_pointwise_forward_f32(
        reinterpret_cast<const float*>(input),
        reinterpret_cast<float*>(output), n_items, op, stream);
  } else {
    static_assert(std::is_same<T, float>::value || sizeof(T) == 2,
                  "supported data types: float and half");
    code = snn_hip_pointwise_forward_f16(input, output, n_items, op, stream);
  }
  return hip::detail::finish(code, stream);
}

// output_backprop[i] = Op'(input_forward[i], input_backprop[i])
// (pointwise/launch.h:120-150).  input_forward is what the reference's tests
// pass: the forward output, or for Log the forward input
// (test/pointwise/pointwise_fixture.h:115-124).
template <typename T, template <typename> class PointwiseType,
          typename Direction, typename Backend,
          typename = internal::EnableIfGradient<Direction>>
SNNStatus launch(
    typename Backend::template pointer_type<T const> input_forward,
    typename Backend::template pointer_type<T const> input_backprop,
    typename Backend::template pointer_type<T> output_backprop,
    size_t const n_items, Backend& backend,
    const std::vector<hip::Event>& events = {}) {
  hipStream_t stream = backend.get_stream();
  hip::detail::wait_for(stream, events);
  constexpr int op = internal::OpCode<PointwiseType>::value;
  int code;
  if (std::is_same<T, float>::value) {
    code = snn_hip_pointwise_grad_f32(
        reinterpret_cast<const float*>(input_forward),
        reinterpret_cast<const float*>(input_backprop),
        reinterpret_cast<float*>(output_backprop), n_items, op, stream);
  } else {
    static_assert(std::is_same<T, float>::value || sizeof(T) == 2,
                  "supported data types: float and half");
    code = snn_hip_pointwise_grad_f16(input_forward, input_backprop,
                                      output_backprop, n_items, op, stream);
  }
  return hip::detail::finish(code, stream);
}

}  // namespace pointwise
}  // namespace sycldnn

#endif  // PORTDNN_HIP_POINTWISE_H_
