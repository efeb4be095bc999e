// Core vocabulary of the sycldnn:: API on the HIP backend: status codes, the
// completion event, layout enumerators and the padding helpers.
//
// The names and meanings are portDNN's (include/portdnn/status.h:31-89,
// padding_mode.h:40, data_format.h:31-43, filter_format.h:32-44,
// batch_format.h:32-44, helpers/padding.h:36-92, helpers/ratio.h:44-79) so
// that code written against portDNN compiles unchanged; the SYCL event is
// replaced by a HIP event recorded on the backend's stream.
#ifndef PORTDNN_HIP_CORE_H_
#define PORTDNN_HIP_CORE_H_

// The HIP runtime API header needs its platform macro when the translation
// unit is compiled by a plain host compiler rather than hipcc.
#ifndef __HIP_PLATFORM_AMD__
#define __HIP_PLATFORM_AMD__ 1
#endif
#include <hip/hip_runtime_api.h>

#include <cstddef>
#include <memory>
#include <stdexcept>
#include <string>
#include <type_traits>
#include <vector>

#include "snn_hip.h"

namespace sycldnn {

enum class StatusCode {
  OK = SNN_HIP_OK,
  InvalidAlgorithm = SNN_HIP_INVALID_ALGORITHM,
  IndexExceeded = SNN_HIP_INDEX_EXCEEDED,
  InsufficientWorkspace = SNN_HIP_INSUFFICIENT_WORKSPACE,
  AllocationProblem = SNN_HIP_ALLOCATION_PROBLEM,
  InvalidParameter = SNN_HIP_INVALID_PARAMETER,
  // Not in portDNN: a HIP runtime call failed (text in snn_hip_last_error()).
  DeviceError = SNN_HIP_DEVICE_ERROR,
};

namespace hip {

// Stand-in for cl::sycl::event: marks the point on the stream after the last
// kernel of a launch.  Copyable; an empty Event is always complete.
class Event {
 public:
  Event() = default;
  static Event record(hipStream_t stream) {
    hipEvent_t ev = nullptr;
    if (hipEventCreateWithFlags(&ev, hipEventDisableTiming) != hipSuccess)
      return Event{};
    if (hipEventRecord(ev, stream) != hipSuccess) {
      (void)hipEventDestroy(ev);
      return Event{};
    }
    Event e;
    e.ev_ = std::shared_ptr<void>(ev, [](void* p) {
      (void)hipEventDestroy(static_cast<hipEvent_t>(p));
    });
    return e;
  }
  void wait() const {
    if (ev_) (void)hipEventSynchronize(static_cast<hipEvent_t>(ev_.get()));
  }
  // Device faults surface here, as asynchronous SYCL errors do through
  // cl::sycl::event::wait_and_throw.
  void wait_and_throw() const {
    if (!ev_) return;
    const hipError_t err =
        hipEventSynchronize(static_cast<hipEvent_t>(ev_.get()));
    if (err != hipSuccess)
      throw std::runtime_error(std::string("HIP error: ") +
                               hipGetErrorString(err));
  }
  hipEvent_t native() const { return static_cast<hipEvent_t>(ev_.get()); }

 private:
  std::shared_ptr<void> ev_;
};

}  // namespace hip

struct SNNStatus {
  SNNStatus(hip::Event e, StatusCode s) : event(std::move(e)), status(s) {}
  SNNStatus(StatusCode s) : status(s) {}  // NOLINT: implicit as in portDNN
  SNNStatus() : status(StatusCode::OK) {}
  // Valid only when status == OK.
  hip::Event event;
  StatusCode status;
};

enum class PaddingMode { VALID, SAME };
enum class DataFormat { NHWC, NCHW };
enum class FilterFormat { HWCF, FCHW, FHWC };
enum class BatchFormat { STRIDED, INTERLEAVED };

namespace helpers {

template <typename Index>
inline Index round_ratio_up(Index num, Index div) {
  static_assert(std::is_integral<Index>::value, "integral types only");
  const Index q = num / div;
  return num < 0 ? q : q + (num % div == 0 ? 0 : 1);
}

template <typename Index>
inline Index round_ratio_up_above_zero(Index num, Index div) {
  static_assert(std::is_integral<Index>::value, "integral types only");
  return num < 0 ? 0 : (num % div != 0 ? num / div + 1 : num / div);
}

template <typename Index>
inline Index round_up_to_nearest_multiple(Index val, Index multiplier) {
  return round_ratio_up_above_zero(val, multiplier) * multiplier;
}

template <typename Index>
struct PaddingAndOutput {
  Index padding;
  Index output;
};

template <typename Index>
PaddingAndOutput<Index> calculate_padding(Index input, Index window,
                                          Index stride, PaddingMode type) {
  if (type == PaddingMode::SAME) {
    const Index out = round_ratio_up(input, stride);
    const Index needed = (out - 1) * stride + window - input;
    return {needed / 2, out};
  }
  return {0, round_ratio_up(input - window + 1, stride)};
}

// Works for Conv2DParams, DepthwiseConv2DParams and PoolingParams.
template <typename Params>
Params add_padding_to(Params params, PaddingMode type) {
  const auto rows = calculate_padding(params.in_rows, params.window_rows,
                                      params.stride_rows, type);
  params.out_rows = rows.output;
  params.pad_rows = rows.padding;
  const auto cols = calculate_padding(params.in_cols, params.window_cols,
                                      params.stride_cols, type);
  params.out_cols = cols.output;
  params.pad_cols = cols.padding;
  return params;
}

}  // namespace helpers

namespace hip {
namespace detail {

// Makes `stream` wait for every dependency, the HIP form of
// cgh.depends_on(events).
inline void wait_for(hipStream_t stream, const std::vector<Event>& events) {
  for (const Event& e : events) {
    if (e.native() != nullptr) (void)hipStreamWaitEvent(stream, e.native(), 0);
  }
}

inline SNNStatus finish(int code, hipStream_t stream) {
  const StatusCode status = static_cast<StatusCode>(code);
  if (status != StatusCode::OK) return status;
  return SNNStatus{Event::record(stream), status};
}

}  // namespace detail
}  // namespace hip
}  // namespace sycldnn

#endif  // PORTDNN_HIP_CORE_H_
