// cuDNN-style layer over the sycldnn:: API on the HIP backend: handle and
// tensor descriptor (include/portdnn/compat/utils.hpp in portDNN, same names
// and meanings; the SYCL queue is replaced by a HIP stream).
#ifndef PORTDNN_COMPAT_UTILS_HPP_
#define PORTDNN_COMPAT_UTILS_HPP_

#include <functional>
#include <memory>
#include <numeric>
#include <vector>

#include "portdnn/hip/backend.h"
#include "portdnn/hip/core.h"

namespace sycldnn {
namespace compat {

// compat/utils.hpp:51.
enum class SNNDataType { SNN_FLOAT = 0, SNN_DOUBLE, SNN_HALF };

// compat/utils.hpp:68-128: owns the backend every compat call runs on.  Work
// is ordered on one stream, as the reference requires an in-order queue.
class SNNHandle {
 public:
  SNNHandle() = default;
  ~SNNHandle() { release(); }
  SNNHandle(const SNNHandle&) = delete;
  SNNHandle& operator=(const SNNHandle&) = delete;

  // stream == nullptr: the handle creates (and later destroys) its own.
  StatusCode init(hipStream_t stream = nullptr) {
    release();
    if (stream == nullptr) {
      if (hipStreamCreate(&stream) != hipSuccess)
        return StatusCode::AllocationProblem;
      owned_ = stream;
    }
    b_.reset(new backend::HIPBackend(stream));
    return StatusCode::OK;
  }
  backend::HIPBackend& getBackend() { return *b_; }
  hipStream_t getStream() const { return b_ ? b_->get_stream() : nullptr; }
  // compat/utils.hpp:110-127 (setQueue).
  StatusCode setStream(hipStream_t stream) {
    if (stream == nullptr) return StatusCode::InvalidParameter;
    release();
    b_.reset(new backend::HIPBackend(stream));
    return StatusCode::OK;
  }

 private:
  void release() {
    b_.reset();
    if (owned_ != nullptr) {
      (void)hipStreamSynchronize(owned_);
      (void)hipStreamDestroy(owned_);
      owned_ = nullptr;
    }
  }
  std::unique_ptr<backend::HIPBackend> b_;
  hipStream_t owned_ = nullptr;
};

// compat/utils.hpp:138-143, :152-154.
inline StatusCode SNNCreate(SNNHandle& handle, hipStream_t stream = nullptr) {
  return handle.init(stream);
}
inline StatusCode queueSet(SNNHandle& handle, hipStream_t stream) {
  return handle.setStream(stream);
}

// compat/utils.hpp:166-203.
class DescriptorBase {
 protected:
  using Index_t = int;
  size_t nDims_;
  std::vector<Index_t> dims_;

 public:
  DescriptorBase() : nDims_(4), dims_(4, 0) {}
  explicit DescriptorBase(int nDims) : nDims_(nDims), dims_(nDims, 0) {}
  virtual ~DescriptorBase() {}
  virtual StatusCode set4d(DataFormat format, int dim0, int dim1, int dim2,
                           int dim3) = 0;
};

// compat/utils.hpp:210-349.  Dimensions are always given as (n, c, h, w);
// `format` says how the data is laid out.  dims_ holds them in storage order.
class TensorDescriptor : public DescriptorBase {
  std::vector<int> stride_;
  DataFormat format_;

 public:
  TensorDescriptor()
      : DescriptorBase(), stride_(4, 1), format_(DataFormat::NCHW) {}
  DataFormat getFormat() const { return format_; }
  size_t getSize() const {
    return std::accumulate(dims_.begin(), dims_.end(), size_t{1},
                           std::multiplies<size_t>());
  }
  StatusCode set4d(DataFormat format, int n, int c, int h,
                   int w) override final {
    if (!(n > 0 && c > 0 && h > 0 && w > 0)) return StatusCode::InvalidParameter;
    nDims_ = 4;
    format_ = format;
    if (format == DataFormat::NCHW) {
      stride_ = {c * h * w, h * w, w, 1};
      dims_ = {n, c, h, w};
    } else if (format == DataFormat::NHWC) {
      stride_ = {c * h * w, 1, w * c, c};
      dims_ = {n, h, w, c};
    } else {
      return StatusCode::InvalidParameter;
    }
    return StatusCode::OK;
  }
  StatusCode get4dDescriptorDims(int* n, int* c, int* h, int* w) const {
    if (n == nullptr || c == nullptr || h == nullptr || w == nullptr)
      return StatusCode::InvalidParameter;
    *n = dims_[0];
    if (format_ == DataFormat::NCHW) {
      *c = dims_[1]; *h = dims_[2]; *w = dims_[3];
    } else {
      *h = dims_[1]; *w = dims_[2]; *c = dims_[3];
    }
    return StatusCode::OK;
  }
  StatusCode get4dDescriptorStride(int* nStride, int* cStride, int* hStride,
                                   int* wStride) const {
    if (nStride == nullptr || cStride == nullptr || hStride == nullptr ||
        wStride == nullptr)
      return StatusCode::InvalidParameter;
    *nStride = stride_[0]; *cStride = stride_[1];
    *hStride = stride_[2]; *wStride = stride_[3];
    return StatusCode::OK;
  }
  StatusCode getTensor4dDescriptor(SNNDataType* dataType, int* n, int* c,
                                   int* h, int* w, int* nStride, int* cStride,
                                   int* hStride, int* wStride) const {
    if (dataType == nullptr) return StatusCode::InvalidParameter;
    *dataType = SNNDataType::SNN_FLOAT;
    const StatusCode st = get4dDescriptorDims(n, c, h, w);
    if (st != StatusCode::OK) return st;
    return get4dDescriptorStride(nStride, cStride, hStride, wStride);
  }
};

// compat/utils.hpp:351-388.
inline StatusCode getTensor4dDescriptor(const TensorDescriptor& tensorDesc,
                                        SNNDataType* dataType, int* n, int* c,
                                        int* h, int* w, int* nStride,
                                        int* cStride, int* hStride,
                                        int* wStride) {
  return tensorDesc.getTensor4dDescriptor(dataType, n, c, h, w, nStride,
                                          cStride, hStride, wStride);
}
inline StatusCode setTensor4dDescriptor(TensorDescriptor& tensorDesc,
                                        DataFormat format, SNNDataType, int n,
                                        int c, int h, int w) {
  return tensorDesc.set4d(format, n, c, h, w);
}

}  // namespace compat
}  // namespace sycldnn

#endif  // PORTDNN_COMPAT_UTILS_HPP_
