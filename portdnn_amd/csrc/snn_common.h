// Shared host/device helpers for libsnn_hip (gfx950 only).
#ifndef PORTDNN_AMD_CSRC_SNN_COMMON_H_
#define PORTDNN_AMD_CSRC_SNN_COMMON_H_

#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <climits>
#include <cstddef>
#include <cstdint>
#include <cstdlib>
#include <string>

#include "snn_hip.h"

namespace snn {

// Records the HIP error text for snn_hip_last_error() and returns
// SNN_HIP_DEVICE_ERROR.
int report_hip_error(hipError_t err, const char* what);

// Records `text` for snn_hip_last_error() and returns `status`.
int report_error(int status, const std::string& text);

#define SNN_HIP_TRY(expr)                                   \
  do {                                                      \
    hipError_t snn_err_ = (expr);                           \
    if (snn_err_ != hipSuccess) {                           \
      return ::snn::report_hip_error(snn_err_, #expr);      \
    }                                                       \
  } while (0)

// Launch-error check placed after every kernel launch.
#define SNN_HIP_CHECK_LAUNCH() SNN_HIP_TRY(hipGetLastError())

// portDNN's SNN_VALIDATE_PARAM (include/portdnn/helpers/macros.h:115-121)
// without the debug assert: a failed condition returns InvalidParameter.
#define SNN_REQUIRE(cond)                         \
  do {                                            \
    if (!(cond)) return SNN_HIP_INVALID_PARAMETER; \
  } while (0)

// Developer switches (tile shapes, kernel choices) are read from the
// environment only in builds made with -DSNN_HIP_TUNING, once per switch; the
// shipped library reads no environment variable and every SNN_TUNING_ENV is a
// null constant the compiler folds away.
#ifdef SNN_HIP_TUNING
#define SNN_TUNING_ENV(name)                     \
  ([]() -> const char* {                         \
    static const char* const value = std::getenv(name); \
    return value;                                \
  }())
#else
#define SNN_TUNING_ENV(name) (static_cast<const char*>(nullptr))
#endif

inline hipStream_t as_stream(void* s) { return static_cast<hipStream_t>(s); }

// Brackets the kernels launched during its lifetime with HIP events on
// `stream` when kernel timing is enabled (snn_hip_kernel_timing_enable);
// otherwise does nothing.
class KernelTimer {
 public:
  explicit KernelTimer(hipStream_t stream);
  ~KernelTimer();
  KernelTimer(const KernelTimer&) = delete;
  KernelTimer& operator=(const KernelTimer&) = delete;

 private:
  hipStream_t stream_;
  hipEvent_t stop_;
};

constexpr int kWave = 64;

inline int ceil_div(int a, int b) { return (a + b - 1) / b; }
inline unsigned ceil_div(unsigned a, unsigned b) { return (a + b - 1) / b; }
inline size_t ceil_div(size_t a, size_t b) { return (a + b - 1) / b; }

// True when a tensor of `elems` elements can be addressed with 32-bit signed
// indices (portDNN returns IndexExceeded otherwise unless built with
// SNN_USE_INT64, src/conv2d/tiled/launch_tiled.cc:133-141).
inline bool fits_int32(size_t elems) {
  return elems <= static_cast<size_t>(INT_MAX);
}

// Element type traits: storage type T, arithmetic in float.
template <typename T>
struct Elem;
template <>
struct Elem<float> {
  __host__ __device__ static float load(const float* p) { return *p; }
  __host__ __device__ static float to_float(float v) { return v; }
  __host__ __device__ static float from_float(float v) { return v; }
};
template <>
struct Elem<_Float16> {
  __host__ __device__ static float load(const _Float16* p) {
    return static_cast<float>(*p);
  }
  __host__ __device__ static float to_float(_Float16 v) {
    return static_cast<float>(v);
  }
  __host__ __device__ static _Float16 from_float(float v) {
    return static_cast<_Float16>(v);
  }
};

// Stream-ordered temporaries (partial results, re-laid-out filters) for calls
// that bring no workspace.  They come from a memory pool of the library's own,
// one per device, that keeps up to 512 MiB of freed blocks instead of handing
// them back at every synchronisation -- the default pool does, and the next
// allocation after a hipStreamSynchronize then costs tens of microseconds.
// Falls back to the device's default pool when a pool cannot be created.
hipError_t temp_malloc_async(void** ptr, size_t bytes, hipStream_t stream);
void temp_free_async(void* ptr, hipStream_t stream);

// Validated, normalised views of the three parameter records.
int validate(const snn_hip_conv2d_params& p);
int validate(const snn_hip_depthwise_params& p);
int validate(const snn_hip_pooling_params& p, bool forward);

}  // namespace snn

#endif  // PORTDNN_AMD_CSRC_SNN_COMMON_H_
