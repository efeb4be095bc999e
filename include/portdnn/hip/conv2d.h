// sycldnn::conv2d on the HIP backend: parameters, tensor sizes, algorithm
// selectors, workspace queries and launch<T, ConvType>.
//
// Mirrors include/portdnn/conv2d/{params,sizes,conv_type,algorithm,
// workspace_size,launch}.h and include/portdnn/conv2d/selector/*.h.  The
// templates only validate and forward to the C ABI in snn_hip.h.
#ifndef PORTDNN_HIP_CONV2D_H_
#define PORTDNN_HIP_CONV2D_H_

#include "portdnn/hip/backend.h"
#include "portdnn/hip/core.h"

namespace sycldnn {
namespace conv2d {

namespace conv_type {
struct Forward {};
struct InputBackprop {};
struct FilterBackprop {};
}  // namespace conv_type

enum class Algorithm {
  NotSupported = SNN_HIP_ALGO_NOT_SUPPORTED,
  Direct = SNN_HIP_ALGO_DIRECT,
  Tiled = SNN_HIP_ALGO_TILED,
  Im2col = SNN_HIP_ALGO_IM2COL,
  Winograd = SNN_HIP_ALGO_WINOGRAD,
  WinogradLarge = SNN_HIP_ALGO_WINOGRAD_LARGE,
  Matmul = SNN_HIP_ALGO_MATMUL,
};

// Field order as in portDNN so that aggregate initialisation carries over.
struct Conv2DParams {
  using Index = int;
  Index channels;
  Index features;
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
  Index dilation_rows = 1;
  Index dilation_cols = 1;
  Index groups = 1;
  sycldnn::DataFormat input_format = sycldnn::DataFormat::NHWC;
  sycldnn::FilterFormat filter_format = sycldnn::FilterFormat::HWCF;
  sycldnn::BatchFormat group_format = sycldnn::BatchFormat::STRIDED;
};

struct ConvSizes {
  size_t input_size;
  size_t filter_size;
  size_t output_size;
};

namespace internal {

template <typename ConvType>
struct Direction;
template <>
struct Direction<conv_type::Forward> {
  static constexpr int value = SNN_HIP_FORWARD;
};
template <>
struct Direction<conv_type::InputBackprop> {
  static constexpr int value = SNN_HIP_INPUT_BACKPROP;
};
template <>
struct Direction<conv_type::FilterBackprop> {
  static constexpr int value = SNN_HIP_FILTER_BACKPROP;
};

inline snn_hip_conv2d_params to_c(Conv2DParams const& p) {
  return {p.channels,      p.features,
          p.batch,         p.in_rows,
          p.in_cols,       p.window_rows,
          p.window_cols,   p.stride_rows,
          p.stride_cols,   p.out_rows,
          p.out_cols,      p.pad_rows,
          p.pad_cols,      p.dilation_rows,
          p.dilation_cols, p.groups,
          static_cast<int>(p.input_format),
          static_cast<int>(p.filter_format),
          static_cast<int>(p.group_format)};
}

}  // namespace internal

// Element counts of (input, filter, output) in the operand roles of the
// direction: FilterBackprop's "filter" is dY and its output is dW.
template <typename ConvType>
inline ConvSizes get_sizes(Conv2DParams const& p) {
  const size_t g = static_cast<size_t>(p.groups > 0 ? p.groups : 1);
  const size_t x = static_cast<size_t>(p.batch) * p.in_rows * p.in_cols *
                   p.channels;
  const size_t w = static_cast<size_t>(p.window_rows) * p.window_cols *
                   p.channels * p.features / g;
  const size_t y = static_cast<size_t>(p.batch) * p.out_rows * p.out_cols *
                   p.features;
  switch (internal::Direction<ConvType>::value) {
    case SNN_HIP_FORWARD:
      return {x, w, y};
    case SNN_HIP_INPUT_BACKPROP:
      return {y, static_cast<size_t>(p.window_rows) * p.window_cols *
                     p.channels * p.features,
              x};
    default:
      return {x, y,
              static_cast<size_t>(p.window_rows) * p.window_cols * p.channels *
                  p.features};
  }
}

// ---- selectors -------------------------------------------------------------

class Selector {
 public:
  virtual ~Selector() = default;
  template <typename ConvType>
  Algorithm select(Conv2DParams const& params) {
    switch (internal::Direction<ConvType>::value) {
      case SNN_HIP_FORWARD:
        return select_forward(params);
      case SNN_HIP_INPUT_BACKPROP:
        return select_input_backprop(params);
      default:
        return select_filter_backprop(params);
    }
  }
  virtual Algorithm select_forward(Conv2DParams const& params) = 0;
  virtual Algorithm select_input_backprop(Conv2DParams const& params) = 0;
  virtual Algorithm select_filter_backprop(Conv2DParams const& params) = 0;
  virtual char const* name() const = 0;
};

namespace internal {
// Selector whose answer is "Algo if libsnn_hip's rule for Algo accepts the
// parameters, NotSupported otherwise" -- the rules are the reference
// selectors', kept in one place behind the C ABI.
template <Algorithm Algo>
class RuleSelector : public Selector {
 public:
  Algorithm select_forward(Conv2DParams const& p) override {
    return ask(p, SNN_HIP_FORWARD);
  }
  Algorithm select_input_backprop(Conv2DParams const& p) override {
    return ask(p, SNN_HIP_INPUT_BACKPROP);
  }
  Algorithm select_filter_backprop(Conv2DParams const& p) override {
    return ask(p, SNN_HIP_FILTER_BACKPROP);
  }

 private:
  static Algorithm ask(Conv2DParams const& p, int direction) {
    const snn_hip_conv2d_params c = to_c(p);
    return static_cast<Algorithm>(snn_hip_conv2d_algorithm_supports(
        &c, direction, static_cast<int>(Algo)));
  }
};
}  // namespace internal

template <Algorithm Algo>
class ConstantSelector final : public internal::RuleSelector<Algo> {
 public:
  char const* name() const override {
    return Algo == Algorithm::Direct   ? "Direct"
           : Algo == Algorithm::Tiled  ? "Tiled"
           : Algo == Algorithm::Im2col ? "Im2col"
                                       : "Constant";
  }
};
using DirectSelector = ConstantSelector<Algorithm::Direct>;
using Im2colSelector = ConstantSelector<Algorithm::Im2col>;

class TiledSelector final : public internal::RuleSelector<Algorithm::Tiled> {
 public:
  char const* name() const override { return "TiledSelector"; }
};
class WinogradSelector final
    : public internal::RuleSelector<Algorithm::Winograd> {
 public:
  char const* name() const override { return "WinogradSelector"; }
};
class WinogradLargeSelector final
    : public internal::RuleSelector<Algorithm::WinogradLarge> {
 public:
  char const* name() const override { return "WinogradLargeSelector"; }
};
class MatmulSelector final : public internal::RuleSelector<Algorithm::Matmul> {
 public:
  char const* name() const override { return "MatmulSelector"; }
};

namespace internal {
template <typename T>
struct DataType {
  static_assert(sizeof(T) == 2, "supported data types: float and half");
  static constexpr int value = SNN_HIP_DTYPE_F16;
};
template <>
struct DataType<float> {
  static constexpr int value = SNN_HIP_DTYPE_F32;
};
}  // namespace internal

// What get_default_selector returns: the per-layer choice tuned for MI355X,
// for float launches unless built for another element type
// (get_default_selector_for<T>): the half-precision kernels are different
// kernels, and half has no Winograd.
class DefaultSelector final : public Selector {
 public:
  explicit DefaultSelector(int dtype = SNN_HIP_DTYPE_F32) : dtype_(dtype) {}
  Algorithm select_forward(Conv2DParams const& p) override {
    return ask(p, SNN_HIP_FORWARD);
  }
  Algorithm select_input_backprop(Conv2DParams const& p) override {
    return ask(p, SNN_HIP_INPUT_BACKPROP);
  }
  Algorithm select_filter_backprop(Conv2DParams const& p) override {
    return ask(p, SNN_HIP_FILTER_BACKPROP);
  }
  char const* name() const override { return "Default"; }

 private:
  Algorithm ask(Conv2DParams const& p, int direction) const {
    const snn_hip_conv2d_params c = internal::to_c(p);
    return static_cast<Algorithm>(
        snn_hip_conv2d_default_algorithm_for(&c, direction, dtype_));
  }
  int dtype_;
};

// portDNN takes a cl::sycl::device here; the HIP build takes the backend (or
// nothing: there is one device kind).
inline std::unique_ptr<Selector> get_default_selector() {
  return std::unique_ptr<Selector>(new DefaultSelector());
}
template <typename Backend>
inline std::unique_ptr<Selector> get_default_selector(Backend const&) {
  return get_default_selector();
}
// Not in portDNN, whose selectors do not know the element type: the default
// selector for launches of element type T.
template <typename T>
inline std::unique_ptr<Selector> get_default_selector_for() {
  return std::unique_ptr<Selector>(
      new DefaultSelector(internal::DataType<T>::value));
}

// ---- workspace ---------------------------------------------------------------

struct WorkspaceSize {
  size_t required_size;     // elements
  size_t recommended_size;  // elements
};

template <typename ConvType>
WorkspaceSize query_workspace_size(Conv2DParams const& params,
                                   Selector& selector) {
  const snn_hip_conv2d_params c = internal::to_c(params);
  const Algorithm algo = selector.select<ConvType>(params);
  WorkspaceSize ws{0, 0};
  (void)snn_hip_conv2d_workspace_size(&c, internal::Direction<ConvType>::value,
                                      static_cast<int>(algo),
                                      &ws.required_size, &ws.recommended_size);
  return ws;
}

// Not in portDNN: the same query for launches of element type T, in elements
// of T.  For half the answer differs from the type-blind one above (required
// is 0, recommended is what the half kernels use).
template <typename T, typename ConvType>
WorkspaceSize query_workspace_size(Conv2DParams const& params,
                                   Selector& selector) {
  const snn_hip_conv2d_params c = internal::to_c(params);
  const Algorithm algo = selector.select<ConvType>(params);
  WorkspaceSize ws{0, 0};
  (void)snn_hip_conv2d_workspace_size_for(
      &c, internal::Direction<ConvType>::value, static_cast<int>(algo),
      internal::DataType<T>::value, &ws.required_size, &ws.recommended_size);
  return ws;
}

// ---- launch ------------------------------------------------------------------

namespace internal {

template <typename T, typename ConvType>
inline int call(T const* input, T const* filter, T* output,
                snn_hip_conv2d_params const& c, int algo, T* workspace,
                size_t workspace_size, hipStream_t stream) {
  constexpr int dir = Direction<ConvType>::value;
  if constexpr (std::is_same<T, float>::value) {
    if (dir == SNN_HIP_FORWARD)
      return snn_hip_conv2d_forward_f32(input, filter, output, &c, algo,
                                        workspace, workspace_size, stream);
    if (dir == SNN_HIP_INPUT_BACKPROP)
      return snn_hip_conv2d_input_backprop_f32(
          input, filter, output, &c, algo, workspace, workspace_size, stream);
    return snn_hip_conv2d_filter_backprop_f32(
        input, filter, output, &c, algo, workspace, workspace_size, stream);
  } else {
    static_assert(sizeof(T) == 2, "supported data types: float and half");
    if (dir == SNN_HIP_FORWARD)
      return snn_hip_conv2d_forward_f16(input, filter, output, &c, algo,
                                        workspace, workspace_size, stream);
    if (dir == SNN_HIP_INPUT_BACKPROP)
      return snn_hip_conv2d_input_backprop_f16(
          input, filter, output, &c, algo, workspace, workspace_size, stream);
    return snn_hip_conv2d_filter_backprop_f16(
        input, filter, output, &c, algo, workspace, workspace_size, stream);
  }
}

}  // namespace internal

// Same parameters and meaning as portDNN's USM launch
// (include/portdnn/conv2d/launch.h:104-118): the workspace is caller-owned and
// counted in elements; `events` are dependencies of the launch.
template <typename T, typename ConvType, typename Backend>
SNNStatus launch(typename Backend::template pointer_type<T const> input,
                 typename Backend::template pointer_type<T const> filter,
                 typename Backend::template pointer_type<T> output,
                 Conv2DParams const& params, Selector& selector,
                 Backend& backend,
                 typename Backend::template pointer_type<T> workspace,
                 size_t workspace_size,
                 const std::vector<hip::Event>& events = {}) {
  const snn_hip_conv2d_params c = internal::to_c(params);
  const Algorithm algo = selector.select<ConvType>(params);
  hipStream_t stream = backend.get_stream();
  hip::detail::wait_for(stream, events);
  return hip::detail::finish(
      internal::call<T, ConvType>(input, filter, output, c,
                                  static_cast<int>(algo), workspace,
                                  workspace_size, stream),
      stream);
}

// Not in portDNN, which runs three launches for this (conv2d::launch,
// binaryop::launch<Add> with the bias as a [features] operand,
// pointwise::launch<Relu, Forward>): output = act(conv(input, filter) +
// bias[feature]) with the bias add and the activation folded into the
// convolution's output stage where the chosen kernel allows it.  `bias` may
// be null.  Forward, float, NHWC only.
enum class Activation {
  None = SNN_HIP_ACTIVATION_NONE,
  Relu = SNN_HIP_ACTIVATION_RELU
};
template <typename T, typename Backend>
SNNStatus launch_forward_bias_activation(
    typename Backend::template pointer_type<T const> input,
    typename Backend::template pointer_type<T const> filter,
    typename Backend::template pointer_type<T const> bias,
    typename Backend::template pointer_type<T> output,
    Conv2DParams const& params, Selector& selector, Backend& backend,
    typename Backend::template pointer_type<T> workspace,
    size_t workspace_size, Activation activation,
    const std::vector<hip::Event>& events = {}) {
  static_assert(std::is_same<T, float>::value,
                "launch_forward_bias_activation is provided for float");
  const snn_hip_conv2d_params c = internal::to_c(params);
  const Algorithm algo = selector.select<conv_type::Forward>(params);
  hipStream_t stream = backend.get_stream();
  hip::detail::wait_for(stream, events);
  return hip::detail::finish(
      snn_hip_conv2d_forward_bias_act_f32(
          input, filter, bias, output, &c, static_cast<int>(algo),
          static_cast<int>(activation), workspace, workspace_size, stream),
      stream);
}

// Not in portDNN, whose Winograd launch transforms the filter every time: a
// launch in two calls for callers that run many launches with one filter.
// prepare_filter writes what the selected algorithm derives from the filter
// alone into the workspace (nothing, for most paths); launch_prepared is
// launch<float, ConvType> trusting those contents.  The caller keeps the
// workspace untouched in between and passes the same filter, parameters and
// selector to both.
template <typename T, typename ConvType, typename Backend>
SNNStatus prepare_filter(
    typename Backend::template pointer_type<T const> filter,
    Conv2DParams const& params, Selector& selector, Backend& backend,
    typename Backend::template pointer_type<T> workspace,
    size_t workspace_size, const std::vector<hip::Event>& events = {}) {
  static_assert(std::is_same<T, float>::value,
                "prepare_filter is provided for float");
  const snn_hip_conv2d_params c = internal::to_c(params);
  const Algorithm algo = selector.select<ConvType>(params);
  hipStream_t stream = backend.get_stream();
  hip::detail::wait_for(stream, events);
  return hip::detail::finish(
      snn_hip_conv2d_prepare_filter_f32(
          internal::Direction<ConvType>::value, filter, &c,
          static_cast<int>(algo), workspace, workspace_size, stream),
      stream);
}
template <typename T, typename ConvType, typename Backend>
SNNStatus launch_prepared(
    typename Backend::template pointer_type<T const> input,
    typename Backend::template pointer_type<T const> filter,
    typename Backend::template pointer_type<T> output,
    Conv2DParams const& params, Selector& selector, Backend& backend,
    typename Backend::template pointer_type<T> workspace,
    size_t workspace_size, const std::vector<hip::Event>& events = {}) {
  static_assert(std::is_same<T, float>::value,
                "launch_prepared is provided for float");
  const snn_hip_conv2d_params c = internal::to_c(params);
  const Algorithm algo = selector.select<ConvType>(params);
  hipStream_t stream = backend.get_stream();
  hip::detail::wait_for(stream, events);
  return hip::detail::finish(
      snn_hip_conv2d_prepared_f32(internal::Direction<ConvType>::value, input,
                                  filter, output, &c, static_cast<int>(algo),
                                  workspace, workspace_size, stream),
      stream);
}

// Not in portDNN, whose kernels always add in one fixed order: the same
// convolution as launch<float, ConvType> with run-to-run bit-identical
// results (no reduction split across work-groups, whose partial sums would
// meet through float atomics in varying order).  Slower for small problems
// and for filter gradients outside the Winograd algorithm.
template <typename T, typename ConvType, typename Backend>
SNNStatus launch_deterministic(
    typename Backend::template pointer_type<T const> input,
    typename Backend::template pointer_type<T const> filter,
    typename Backend::template pointer_type<T> output,
    Conv2DParams const& params, Selector& selector, Backend& backend,
    typename Backend::template pointer_type<T> workspace,
    size_t workspace_size, const std::vector<hip::Event>& events = {}) {
  static_assert(std::is_same<T, float>::value,
                "launch_deterministic is provided for float");
  const snn_hip_conv2d_params c = internal::to_c(params);
  const Algorithm algo = selector.select<ConvType>(params);
  hipStream_t stream = backend.get_stream();
  hip::detail::wait_for(stream, events);
  return hip::detail::finish(
      snn_hip_conv2d_deterministic_f32(
          internal::Direction<ConvType>::value, input, filter, output, &c,
          static_cast<int>(algo), workspace, workspace_size, stream),
      stream);
}

}  // namespace conv2d
}  // namespace sycldnn

#endif  // PORTDNN_HIP_CONV2D_H_
