// sycldnn::backend::HIPBackend -- the backend object the launch templates take.
//
// It plays the role portDNN's SNNUSMBackend plays for SYCL USM pointers
// (include/portdnn/backend/snn_usm_backend.h:60-163): plain T* device
// pointers, allocate / deallocate for internal scratch, and the matmul /
// batch_matmul members of the backend concept
// (include/portdnn/backend/backend_interface.h:93-118), here served by
// libsnn_hip's MFMA GEMM.  Work is ordered on one HIP stream per backend
// object.  Launches from different backends do not share mutable state except
// the library's per-device pool of stream-ordered temporaries (thread-safe)
// and, for the one no-allocation depthwise entry point, its scratch array
// (calls that overlap on one GPU race on it, as its declaration says).
#ifndef PORTDNN_HIP_BACKEND_H_
#define PORTDNN_HIP_BACKEND_H_

#include "portdnn/hip/core.h"

namespace sycldnn {
namespace backend {

class HIPBackend {
 public:
  template <typename T>
  using pointer_type = T*;
  template <typename T>
  using internal_pointer_type = T*;

  // Uses `stream` for every launch (nullptr = the default stream).  The
  // stream stays owned by the caller.
  explicit HIPBackend(hipStream_t stream = nullptr) : stream_(stream) {}

  static char const* name() { return "HIPBackend"; }
  hipStream_t get_stream() const { return stream_; }

  template <typename T>
  T* allocate(size_t n_elems) {
    void* p = nullptr;
    if (hipMalloc(&p, n_elems * sizeof(T)) != hipSuccess) return nullptr;
    return static_cast<T*>(p);
  }
  template <typename T>
  void deallocate(T* ptr) {
    (void)hipFree(const_cast<typename std::remove_const<T>::type*>(ptr));
  }

  // The external -> internal pointer conversions of the backend concept are
  // identities here.
  template <typename T>
  T* to_internal_pointer(T* ptr) { return ptr; }
  template <typename T>
  void release_internal_pointer(T*) {}

  // output = op(lhs) * op(rhs) + beta * output, row-major, op(lhs) m x k and
  // op(rhs) k x n.
  template <bool TransposeLHS, bool TransposeRHS, typename Index>
  hip::Event matmul(float const* lhs, float const* rhs, float* output,
                    float beta, Index m, Index k, Index n,
                    const std::vector<hip::Event>& events = {}) {
    return batch_matmul<TransposeLHS, TransposeRHS>(lhs, rhs, output, Index{1},
                                                    m, k, n, beta, events);
  }
  template <bool TransposeLHS, bool TransposeRHS, typename Index>
  hip::Event batch_matmul(float const* lhs, float const* rhs, float* output,
                          Index n_batches, Index m, Index k, Index n,
                          float beta = 0.f,
                          const std::vector<hip::Event>& events = {}) {
    hip::detail::wait_for(stream_, events);
    const int code = snn_hip_matmul_f32(
        lhs, rhs, output, static_cast<int>(n_batches), static_cast<int>(m),
        static_cast<int>(k), static_cast<int>(n), TransposeLHS, TransposeRHS,
        beta, stream_);
    if (code != SNN_HIP_OK)
      throw std::runtime_error(std::string("matmul failed: ") +
                               snn_hip_status_string(code));
    return hip::Event::record(stream_);
  }

 private:
  hipStream_t stream_;
};

}  // namespace backend
}  // namespace sycldnn

#endif  // PORTDNN_HIP_BACKEND_H_
