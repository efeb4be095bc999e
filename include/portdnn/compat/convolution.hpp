// cuDNN-style layer over sycldnn::conv2d on the HIP backend: descriptors and
// convolutionForward / BackwardData / BackwardFilter with alpha / beta
// scaling (include/portdnn/compat/convolution.hpp and compat/scaling.hpp in
// portDNN, same names and meanings).
//
// result = alpha * conv(...) + beta * (what the output held before).  A zero
// alpha skips the convolution, a zero beta ignores the previous contents
// (compat/scaling.hpp:96-262).  NHWC / HWCF descriptors run on any
// algorithm; NCHW / FCHW descriptors are served by Algorithm::Direct only, as
// in the reference (internal/conv2d/launch.h:191-194).  Grouped convolutions
// give InvalidAlgorithm.
#ifndef PORTDNN_COMPAT_CONVOLUTION_HPP_
#define PORTDNN_COMPAT_CONVOLUTION_HPP_

#include <cmath>
#include <memory>
#include <vector>

#include "portdnn/compat/utils.hpp"
#include "portdnn/hip/conv2d.h"
#include "snn_hip.h"

namespace sycldnn {
namespace compat {

// compat/convolution.hpp:46-51.
enum class ConvolutionMode { CONVOLUTION = 0, CROSS_CORRELATION };

// compat/convolution.hpp:57-205.
class ConvolutionDescriptor {
  using Index_t = int;
  size_t nDims_;
  std::vector<Index_t> padding_;
  std::vector<Index_t> stride_;
  std::vector<Index_t> dilation_;
  ConvolutionMode mode_ = ConvolutionMode::CROSS_CORRELATION;
  Index_t groupCount_ = 1;

 public:
  ConvolutionDescriptor()
      : nDims_(2), padding_(2, 0), stride_(2, 1), dilation_(2, 1) {}
  size_t getNumDims() const { return nDims_; }
  std::vector<Index_t> getPadding() const { return padding_; }
  std::vector<Index_t> getStride() const { return stride_; }
  std::vector<Index_t> getDilation() const { return dilation_; }
  ConvolutionMode getMode() const { return mode_; }
  Index_t getStrideH() const { return stride_[0]; }
  Index_t getStrideW() const { return stride_[1]; }
  Index_t getPadH() const { return padding_[0]; }
  Index_t getPadW() const { return padding_[1]; }
  Index_t getDilationH() const { return dilation_[0]; }
  Index_t getDilationW() const { return dilation_[1]; }
  Index_t getGroupCount() const { return groupCount_; }
  StatusCode setGroupCount(int groupCount) {
    if (groupCount <= 0) return StatusCode::InvalidParameter;
    groupCount_ = groupCount;
    return StatusCode::OK;
  }
  StatusCode set2d(int pad_h, int pad_w, int stride_h, int stride_w,
                   int dilation_h, int dilation_w,
                   ConvolutionMode mode = ConvolutionMode::CROSS_CORRELATION) {
    return setNd({pad_h, pad_w}, {stride_h, stride_w},
                 {dilation_h, dilation_w}, mode);
  }
  StatusCode setNd(const std::vector<int>& pads,
                   const std::vector<int>& strides,
                   const std::vector<int>& dilations,
                   ConvolutionMode mode = ConvolutionMode::CROSS_CORRELATION) {
    if (pads.size() != strides.size() || pads.size() != dilations.size())
      return StatusCode::InvalidParameter;
    for (int pad : pads)
      if (pad < 0) return StatusCode::InvalidParameter;
    for (int stride : strides)
      if (stride <= 0) return StatusCode::InvalidParameter;
    for (int dilation : dilations)
      if (dilation < 1) return StatusCode::InvalidParameter;
    // Only cross-correlation is supported, as in the reference.
    if (mode != ConvolutionMode::CROSS_CORRELATION)
      return StatusCode::InvalidParameter;
    nDims_ = pads.size();
    padding_ = pads;
    stride_ = strides;
    dilation_ = dilations;
    mode_ = mode;
    return StatusCode::OK;
  }
};

// compat/convolution.hpp:222-273.
inline StatusCode setConvolution2dDescriptor(ConvolutionDescriptor& desc,
                                             int pad_h, int pad_w, int stride_h,
                                             int stride_w, int dilation_h,
                                             int dilation_w,
                                             ConvolutionMode mode) {
  return desc.set2d(pad_h, pad_w, stride_h, stride_w, dilation_h, dilation_w,
                    mode);
}
inline StatusCode setConvolutionNdDescriptor(ConvolutionDescriptor& desc,
                                             int num_spatial_dims,
                                             const int* pads,
                                             const int* strides,
                                             const int* dilations,
                                             ConvolutionMode mode) {
  if (num_spatial_dims != 2) return StatusCode::InvalidParameter;
  return desc.setNd(std::vector<int>(pads, pads + 2),
                    std::vector<int>(strides, strides + 2),
                    std::vector<int>(dilations, dilations + 2), mode);
}
inline StatusCode setConvolutionGroupCount(ConvolutionDescriptor& desc,
                                           int groupCount) {
  return desc.setGroupCount(groupCount);
}

// compat/convolution.hpp:279-381.  Dimensions are always given as
// (k, c, h, w); NCHW stores the filter as FCHW, NHWC as HWCF.
class FilterDescriptor : public DescriptorBase {
  FilterFormat format_ = FilterFormat::FCHW;

 public:
  FilterDescriptor() : DescriptorBase() {}
  explicit FilterDescriptor(size_t nDims)
      : DescriptorBase(static_cast<int>(nDims)) {}
  FilterFormat getFormat() const { return format_; }
  size_t getSize() const {
    return std::accumulate(dims_.begin(), dims_.end(), size_t{1},
                           std::multiplies<size_t>());
  }
  StatusCode set4d(DataFormat format, int k, int c, int h,
                   int w) override final {
    if (!(k > 0 && c > 0 && h > 0 && w > 0)) return StatusCode::InvalidParameter;
    nDims_ = 4;
    if (format == DataFormat::NCHW) {
      format_ = FilterFormat::FCHW;
      dims_ = {k, c, h, w};
    } else if (format == DataFormat::NHWC) {
      format_ = FilterFormat::HWCF;
      dims_ = {h, w, c, k};
    } else {
      return StatusCode::InvalidParameter;
    }
    return StatusCode::OK;
  }
  StatusCode get4dDescriptorDims(int* k, int* c, int* h, int* w) const {
    if (k == nullptr || c == nullptr || h == nullptr || w == nullptr)
      return StatusCode::InvalidParameter;
    if (format_ == FilterFormat::FCHW) {
      *k = dims_[0]; *c = dims_[1]; *h = dims_[2]; *w = dims_[3];
    } else {
      *h = dims_[0]; *w = dims_[1]; *c = dims_[2]; *k = dims_[3];
    }
    return StatusCode::OK;
  }
  StatusCode getFilter4dDescriptor(SNNDataType* dataType, FilterFormat* format,
                                   int* k, int* c, int* h, int* w) const {
    if (dataType == nullptr || format == nullptr)
      return StatusCode::InvalidParameter;
    *dataType = SNNDataType::SNN_FLOAT;
    *format = format_;
    return get4dDescriptorDims(k, c, h, w);
  }
};

// compat/convolution.hpp:384-389, :918-923.
inline StatusCode getFilter4dDescriptor(const FilterDescriptor& filterDesc,
                                        SNNDataType* dataType,
                                        FilterFormat* format, int* k, int* c,
                                        int* h, int* w) {
  return filterDesc.getFilter4dDescriptor(dataType, format, k, c, h, w);
}
inline StatusCode setFilter4dDescriptor(FilterDescriptor& filterDesc,
                                        SNNDataType, DataFormat format, int k,
                                        int c, int h, int w) {
  return filterDesc.set4d(format, k, c, h, w);
}

// compat/convolution.hpp:403-437: out = 1 + (in + 2 pad - ((filter - 1) *
// dilation + 1)) / stride per spatial dimension.
inline StatusCode getConvolution2dForwardOutputDim(
    const ConvolutionDescriptor& desc, const TensorDescriptor& in,
    const FilterDescriptor& filt, int* n, int* c, int* h, int* w) {
  if (n == nullptr || c == nullptr || h == nullptr || w == nullptr)
    return StatusCode::InvalidParameter;
  int inN, inC, inH, inW, fK, fC, fH, fW;
  in.get4dDescriptorDims(&inN, &inC, &inH, &inW);
  filt.get4dDescriptorDims(&fK, &fC, &fH, &fW);
  auto newDim = [](int input, int filter, int pad, int dilation, int stride) {
    return 1 + (input + 2 * pad - ((filter - 1) * dilation + 1)) / stride;
  };
  *n = inN;
  *c = fK;
  *h = newDim(inH, fH, desc.getPadH(), desc.getDilationH(), desc.getStrideH());
  *w = newDim(inW, fW, desc.getPadW(), desc.getDilationW(), desc.getStrideW());
  return StatusCode::OK;
}

namespace internal {

// compat/convolution.hpp:444-505.
inline conv2d::Conv2DParams descToSnnParams(
    const TensorDescriptor& xDesc, const TensorDescriptor& yDesc,
    const FilterDescriptor& wDesc, const ConvolutionDescriptor& convDesc) {
  int inN, inC, inH, inW, fK, fC, fH, fW, outN, outC, outH, outW;
  xDesc.get4dDescriptorDims(&inN, &inC, &inH, &inW);
  wDesc.get4dDescriptorDims(&fK, &fC, &fH, &fW);
  yDesc.get4dDescriptorDims(&outN, &outC, &outH, &outW);
  conv2d::Conv2DParams p{};
  p.channels = inC;
  p.features = fK;
  p.batch = inN;
  p.in_rows = inH;
  p.in_cols = inW;
  p.window_rows = fH;
  p.window_cols = fW;
  p.stride_rows = convDesc.getStrideH();
  p.stride_cols = convDesc.getStrideW();
  p.out_rows = outH;
  p.out_cols = outW;
  p.pad_rows = convDesc.getPadH();
  p.pad_cols = convDesc.getPadW();
  p.dilation_rows = convDesc.getDilationH();
  p.dilation_cols = convDesc.getDilationW();
  p.filter_format = wDesc.getFormat();
  p.input_format = xDesc.getFormat();
  p.groups = convDesc.getGroupCount();
  return p;
}

// compat/convolution.hpp:507-523.
inline std::unique_ptr<conv2d::Selector> getSelector(conv2d::Algorithm algo) {
  using A = conv2d::Algorithm;
  switch (algo) {
    case A::Im2col:
      return std::unique_ptr<conv2d::Selector>(new conv2d::Im2colSelector());
    case A::Winograd:
      return std::unique_ptr<conv2d::Selector>(new conv2d::WinogradSelector());
    case A::Tiled:
      return std::unique_ptr<conv2d::Selector>(new conv2d::TiledSelector());
    case A::Matmul:
      return std::unique_ptr<conv2d::Selector>(new conv2d::MatmulSelector());
    case A::Direct:
      return std::unique_ptr<conv2d::Selector>(new conv2d::DirectSelector());
    default:
      return nullptr;
  }
}

template <typename ConvType>
conv2d::WorkspaceSize getConvolutionWorkspaceSize(
    const TensorDescriptor& xDesc, const FilterDescriptor& wDesc,
    const ConvolutionDescriptor& convDesc, const TensorDescriptor& yDesc,
    conv2d::Algorithm algo) {
  const conv2d::Conv2DParams p = descToSnnParams(xDesc, yDesc, wDesc, convDesc);
  std::unique_ptr<conv2d::Selector> selector = getSelector(algo);
  if (!selector) return conv2d::WorkspaceSize{0, 0};
  return conv2d::query_workspace_size<ConvType>(p, *selector);
}

inline bool isSame(float a, float b) { return std::fabs(a - b) < 1e-9f; }

// The three convolution entry points share everything but the direction and
// which descriptor describes the output (`out_size` elements at `out`).
template <typename ValueT, typename ConvType>
SNNStatus scaledConvolution(SNNHandle& handle, const ValueT* alpha,
                            const ValueT* beta, const void* in,
                            const void* fil, void* out, size_t out_size,
                            const conv2d::Conv2DParams& params,
                            conv2d::Algorithm algo, void* workSpace,
                            size_t workSpaceSizeInBytes) {
  static_assert(std::is_same<ValueT, float>::value,
                "the compat layer is provided for float");
  if (alpha == nullptr || beta == nullptr || out == nullptr)
    return SNNStatus(StatusCode::InvalidParameter);
  std::unique_ptr<conv2d::Selector> selector = getSelector(algo);
  if (!selector) return SNNStatus(StatusCode::InvalidParameter);
  backend::HIPBackend& backend = handle.getBackend();
  hipStream_t stream = backend.get_stream();
  float* y = static_cast<float*>(out);
  const float a = *alpha, b = *beta;
  if (isSame(a, 0.f)) {
    // compat/scaling.hpp:113-121, :166-171: no convolution; y = beta * y.
    if (isSame(b, 1.f)) return hip::detail::finish(SNN_HIP_OK, stream);
    return hip::detail::finish(
        snn_hip_scale_blend_f32(y, nullptr, isSame(b, 0.f) ? 0.f : b, 0.f,
                                out_size, stream),
        stream);
  }
  // compat/scaling.hpp:129-134: the previous output is kept aside when it
  // takes part in the result.
  float* prior = nullptr;
  if (!isSame(b, 0.f)) {
    if (hipMallocAsync(reinterpret_cast<void**>(&prior),
                       out_size * sizeof(float), stream) != hipSuccess)
      return SNNStatus(StatusCode::AllocationProblem);
    (void)hipMemcpyAsync(prior, y, out_size * sizeof(float),
                         hipMemcpyDeviceToDevice, stream);
  }
  SNNStatus status = conv2d::launch<float, ConvType>(
      static_cast<const float*>(in), static_cast<const float*>(fil), y, params,
      *selector, backend, static_cast<float*>(workSpace),
      workSpaceSizeInBytes / sizeof(float));
  if (status.status == StatusCode::OK &&
      !(isSame(a, 1.f) && isSame(b, 0.f)))
    status = hip::detail::finish(
        snn_hip_scale_blend_f32(y, prior, a, prior ? b : 0.f, out_size,
                                stream),
        stream);
  if (prior != nullptr) (void)hipFreeAsync(prior, stream);
  return status;
}

}  // namespace internal

// compat/convolution.hpp:704-732.
template <typename ValueT>
SNNStatus convolutionForward(SNNHandle& handle, const ValueT* alpha,
                             const TensorDescriptor& xDesc, const void* x,
                             const FilterDescriptor& wDesc, const void* w,
                             const ConvolutionDescriptor& convDesc,
                             conv2d::Algorithm algo, void* workSpace,
                             size_t workSpaceSizeInBytes, const ValueT* beta,
                             const TensorDescriptor& yDesc, void* y) {
  return internal::scaledConvolution<ValueT, conv2d::conv_type::Forward>(
      handle, alpha, beta, x, w, y, yDesc.getSize(),
      internal::descToSnnParams(xDesc, yDesc, wDesc, convDesc), algo,
      workSpace, workSpaceSizeInBytes);
}

// compat/convolution.hpp:824-851: dx = alpha * conv_backward_data(dy, w) +
// beta * dx.
template <typename ValueT>
SNNStatus convolutionBackwardData(SNNHandle& handle, const ValueT* alpha,
                                  const FilterDescriptor& wDesc, const void* w,
                                  const TensorDescriptor& dyDesc,
                                  const void* dy,
                                  const ConvolutionDescriptor& convDesc,
                                  conv2d::Algorithm algo, void* workSpace,
                                  size_t workSpaceSizeInBytes,
                                  const ValueT* beta,
                                  const TensorDescriptor& dxDesc, void* dx) {
  return internal::scaledConvolution<ValueT, conv2d::conv_type::InputBackprop>(
      handle, alpha, beta, dy, w, dx, dxDesc.getSize(),
      internal::descToSnnParams(dxDesc, dyDesc, wDesc, convDesc), algo,
      workSpace, workSpaceSizeInBytes);
}

// compat/convolution.hpp:874-901: dw = alpha * conv_backward_filter(x, dy) +
// beta * dw.
template <typename ValueT>
SNNStatus convolutionBackwardFilter(
    SNNHandle& handle, const ValueT* alpha, const TensorDescriptor& xDesc,
    const void* x, const TensorDescriptor& dyDesc, const void* dy,
    const ConvolutionDescriptor& convDesc, conv2d::Algorithm algo,
    void* workSpace, size_t workSpaceSizeInBytes, const ValueT* beta,
    const FilterDescriptor& dwDesc, void* dw) {
  return internal::scaledConvolution<ValueT,
                                     conv2d::conv_type::FilterBackprop>(
      handle, alpha, beta, x, dy, dw, dwDesc.getSize(),
      internal::descToSnnParams(xDesc, dyDesc, dwDesc, convDesc), algo,
      workSpace, workSpaceSizeInBytes);
}

// compat/convolution.hpp:746-815: workspace sizes in bytes (the recommended
// size of query_workspace_size).
inline StatusCode getConvolutionForwardWorkspaceSize(
    SNNHandle&, const TensorDescriptor& xDesc, const FilterDescriptor& wDesc,
    const ConvolutionDescriptor& convDesc, const TensorDescriptor& yDesc,
    conv2d::Algorithm algo, size_t* workSpaceSizeInBytes) {
  if (workSpaceSizeInBytes == nullptr) return StatusCode::InvalidParameter;
  *workSpaceSizeInBytes =
      internal::getConvolutionWorkspaceSize<conv2d::conv_type::Forward>(
          xDesc, wDesc, convDesc, yDesc, algo)
          .recommended_size *
      sizeof(float);
  return StatusCode::OK;
}
inline StatusCode getConvolutionBackwardFilterWorkspaceSize(
    SNNHandle&, const TensorDescriptor& xDesc, const TensorDescriptor& dyDesc,
    const ConvolutionDescriptor& convDesc, const FilterDescriptor& dwDesc,
    conv2d::Algorithm algo, size_t* workSpaceSizeInBytes) {
  if (workSpaceSizeInBytes == nullptr) return StatusCode::InvalidParameter;
  *workSpaceSizeInBytes =
      internal::getConvolutionWorkspaceSize<conv2d::conv_type::FilterBackprop>(
          xDesc, dwDesc, convDesc, dyDesc, algo)
          .recommended_size *
      sizeof(float);
  return StatusCode::OK;
}
inline StatusCode getConvolutionBackwardDataWorkspaceSize(
    SNNHandle&, const FilterDescriptor& wDesc, const TensorDescriptor& dyDesc,
    const ConvolutionDescriptor& convDesc, const TensorDescriptor& dxDesc,
    conv2d::Algorithm algo, size_t* workSpaceSizeInBytes) {
  if (workSpaceSizeInBytes == nullptr) return StatusCode::InvalidParameter;
  *workSpaceSizeInBytes =
      internal::getConvolutionWorkspaceSize<conv2d::conv_type::InputBackprop>(
          dxDesc, wDesc, convDesc, dyDesc, algo)
          .recommended_size *
      sizeof(float);
  return StatusCode::OK;
}

}  // namespace compat
}  // namespace sycldnn

#endif  // PORTDNN_COMPAT_CONVOLUTION_HPP_
