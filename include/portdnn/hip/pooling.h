// sycldnn::pooling on the HIP backend
// (include/portdnn/pooling/{params,sizes,operators,launch}.h).
#ifndef PORTDNN_HIP_POOLING_H_
#define PORTDNN_HIP_POOLING_H_

#include "portdnn/hip/backend.h"
#include "portdnn/hip/core.h"

namespace sycldnn {
namespace pooling {

struct PoolingParams {
  using Index = int;
  Index in_rows;
  Index in_cols;
  Index out_rows;
  Index out_cols;
  Index window_rows;
  Index window_cols;
  Index stride_rows;
  Index stride_cols;
  Index batch;
  Index channels;
  Index pad_rows;
  Index pad_cols;
  sycldnn::DataFormat input_format = sycldnn::DataFormat::NHWC;
};

// Operator and direction tags.  The operators are templates on the data type
// in portDNN and are used as template template arguments; they carry no state
// on the host.
template <typename T>
struct Max {};
template <typename T>
struct MaxWithNan {};
template <typename T>
struct Average {};
struct Forward {};
struct Backpropagate {};

struct PoolingSizes {
  size_t input_size;
  size_t output_size;
};

template <typename Direction>
inline PoolingSizes get_sizes(PoolingParams const& p) {
  const size_t x = static_cast<size_t>(p.batch) * p.in_rows * p.in_cols *
                   p.channels;
  const size_t y = static_cast<size_t>(p.batch) * p.out_rows * p.out_cols *
                   p.channels;
  if (std::is_same<Direction, Forward>::value) return {x, y};
  return {y, x};
}

namespace internal {

template <template <typename> class Op>
struct OpCode;
template <>
struct OpCode<Max> {
  static constexpr int value = SNN_HIP_POOL_MAX;
};
template <>
struct OpCode<MaxWithNan> {
  static constexpr int value = SNN_HIP_POOL_MAX_WITH_NAN;
};
template <>
struct OpCode<Average> {
  static constexpr int value = SNN_HIP_POOL_AVERAGE;
};

template <typename T, template <typename> class Op, typename Direction>
struct IsMaxGradient {
  static constexpr bool value =
      std::is_same<Direction, Backpropagate>::value &&
      OpCode<Op>::value != SNN_HIP_POOL_AVERAGE;
};

inline snn_hip_pooling_params to_c(PoolingParams const& p) {
  return {p.in_rows,     p.in_cols,     p.out_rows,    p.out_cols,
          p.window_rows, p.window_cols, p.stride_rows, p.stride_cols,
          p.batch,       p.channels,    p.pad_rows,    p.pad_cols,
          static_cast<int>(p.input_format)};
}

}  // namespace internal

// Forward (any operator) and the Average gradient: two tensors.
template <typename T, template <typename> class PoolType, typename Direction,
          typename Backend,
          typename = typename std::enable_if<
              !internal::IsMaxGradient<T, PoolType, Direction>::value>::type>
SNNStatus launch(typename Backend::template pointer_type<T const> input,
                 typename Backend::template pointer_type<T> output,
                 PoolingParams const& pp, Backend& backend,
                 const std::vector<hip::Event>& events = {}) {
  const snn_hip_pooling_params c = internal::to_c(pp);
  hipStream_t stream = backend.get_stream();
  hip::detail::wait_for(stream, events);
  int code;
  if constexpr (std::is_same<Direction, Forward>::value) {
    if constexpr (std::is_same<T, float>::value) {
      code = snn_hip_pooling_forward_f32(
          input, output, &c, internal::OpCode<PoolType>::value, stream);
    } else {
      static_assert(sizeof(T) == 2, "supported data types: float and half");
      code = snn_hip_pooling_forward_f16(
          input, output, &c, internal::OpCode<PoolType>::value, stream);
    }
  } else if constexpr (std::is_same<T, float>::value) {
    code = snn_hip_pooling_avg_grad_f32(input, output, &c, stream);
  } else {
    static_assert(sizeof(T) == 2, "supported data types: float and half");
    code = snn_hip_pooling_avg_grad_f16(input, output, &c, stream);
  }
  return hip::detail::finish(code, stream);
}

// Max / MaxWithNan gradient: forward input and output, dY, dX.
template <typename T, template <typename> class PoolType, typename Direction,
          typename Backend,
          typename = typename std::enable_if<
              internal::IsMaxGradient<T, PoolType, Direction>::value>::type>
SNNStatus launch(typename Backend::template pointer_type<T const> input_data,
                 typename Backend::template pointer_type<T const> output_data,
                 typename Backend::template pointer_type<T const> input_backprop,
                 typename Backend::template pointer_type<T> output_backprop,
                 PoolingParams const& pp, Backend& backend,
                 const std::vector<hip::Event>& events = {}) {
  const snn_hip_pooling_params c = internal::to_c(pp);
  hipStream_t stream = backend.get_stream();
  hip::detail::wait_for(stream, events);
  int code;
  if constexpr (std::is_same<T, float>::value) {
    code = snn_hip_pooling_max_grad_f32(input_data, output_data,
                                        input_backprop, output_backprop, &c,
                                        internal::OpCode<PoolType>::value,
                                        stream);
  } else {
    static_assert(sizeof(T) == 2, "supported data types: float and half");
    code = snn_hip_pooling_max_grad_f16(input_data, output_data,
                                        input_backprop, output_backprop, &c,
                                        internal::OpCode<PoolType>::value,
                                        stream);
  }
  return hip::detail::finish(code, stream);
}

}  // namespace pooling
}  // namespace sycldnn

#endif  // PORTDNN_HIP_POOLING_H_
