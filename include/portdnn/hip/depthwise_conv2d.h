// sycldnn::depthwise_conv2d on the HIP backend
// (include/portdnn/depthwise_conv2d/{params,sizes,launch}.h).
#ifndef PORTDNN_HIP_DEPTHWISE_CONV2D_H_
#define PORTDNN_HIP_DEPTHWISE_CONV2D_H_

#include "portdnn/hip/conv2d.h"

namespace sycldnn {
namespace depthwise_conv2d {

struct DepthwiseConv2DParams {
  using Index = int;
  Index channels;
  Index channel_multiplier;
  Index batch;
  Index in_rows;
  Index in_cols;
  Index window_rows;
  Index window_cols;
  Index stride_rows;
  Index stride_cols;
  Index out_rows;
  Index out_cols;
  Index pad_rows;
  Index pad_cols;
  sycldnn::DataFormat input_format = sycldnn::DataFormat::NHWC;
  sycldnn::FilterFormat filter_format = sycldnn::FilterFormat::HWCF;
};

struct ConvSizes {
  size_t input_size;
  size_t filter_size;
  size_t output_size;
};

template <typename ConvType>
inline ConvSizes get_sizes(DepthwiseConv2DParams const& p) {
  const size_t x = static_cast<size_t>(p.batch) * p.in_rows * p.in_cols *
                   p.channels;
  const size_t w = static_cast<size_t>(p.window_rows) * p.window_cols *
                   p.channels * p.channel_multiplier;
  const size_t y = static_cast<size_t>(p.batch) * p.out_rows * p.out_cols *
                   p.channels * p.channel_multiplier;
  switch (conv2d::internal::Direction<ConvType>::value) {
    case SNN_HIP_FORWARD:
      return {x, w, y};
    case SNN_HIP_INPUT_BACKPROP:
      return {y, w, x};
    default:
      return {x, y, w};
  }
}

template <typename T, typename ConvType, typename Backend>
SNNStatus launch(typename Backend::template pointer_type<T const> input,
                 typename Backend::template pointer_type<T const> filter,
                 typename Backend::template pointer_type<T> output,
                 DepthwiseConv2DParams const& p, Backend& backend,
                 const std::vector<hip::Event>& events = {}) {
  const snn_hip_depthwise_params c = {
      p.channels,    p.channel_multiplier, p.batch,       p.in_rows,
      p.in_cols,     p.window_rows,        p.window_cols, p.stride_rows,
      p.stride_cols, p.out_rows,           p.out_cols,    p.pad_rows,
      p.pad_cols,    static_cast<int>(p.input_format),
      static_cast<int>(p.filter_format)};
  hipStream_t stream = backend.get_stream();
  hip::detail::wait_for(stream, events);
  constexpr int dir = conv2d::internal::Direction<ConvType>::value;
  int code;
  if constexpr (std::is_same<T, float>::value) {
    code = dir == SNN_HIP_FORWARD
               ? snn_hip_depthwise_conv2d_forward_f32(input, filter, output,
                                                      &c, stream)
           : dir == SNN_HIP_INPUT_BACKPROP
               ? snn_hip_depthwise_conv2d_input_backprop_f32(
                     input, filter, output, &c, stream)
               : snn_hip_depthwise_conv2d_filter_backprop_f32(
                     input, filter, output, &c, stream);
  } else {
    static_assert(sizeof(T) == 2, "supported data types: float and half");
    code = dir == SNN_HIP_FORWARD
               ? snn_hip_depthwise_conv2d_forward_f16(input, filter, output,
                                                      &c, stream)
           : dir == SNN_HIP_INPUT_BACKPROP
               ? snn_hip_depthwise_conv2d_input_backprop_f16(
                     input, filter, output, &c, stream)
               : snn_hip_depthwise_conv2d_filter_backprop_f16(
                     input, filter, output, &c, stream);
  }
  return hip::detail::finish(code, stream);
}

}  // namespace depthwise_conv2d
}  // namespace sycldnn

#endif  // PORTDNN_HIP_DEPTHWISE_CONV2D_H_
