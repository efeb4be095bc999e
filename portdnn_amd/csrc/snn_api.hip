// The C ABI of libsnn_hip.so: parameter validation, algorithm support rules,
// workspace sizing and dispatch to the kernel launchers.
#include <atomic>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <string>
#include <type_traits>
#include <utility>
#include <vector>

#include "snn_kernels.h"

namespace snn {

namespace {
thread_local std::string g_last_error;
}

// Process-wide state of the library: this opt-in kernel-timing record, the
// per-device memory pool for stream-ordered temporaries below (created at
// first use, kept until the process ends) and the scratch array of the
// no-allocation depthwise entry point (depthwise.hip).
// The timing switch is atomic and the list of event pairs is guarded by a
// mutex, so launches from several threads may record concurrently; the list
// stops growing at kMaxTimedKernels pairs until it is read.
namespace {
std::atomic<bool> g_timing_enabled{false};
std::mutex g_timing_mutex;
std::vector<std::pair<hipEvent_t, hipEvent_t>> g_timed_kernels;
constexpr size_t kMaxTimedKernels = 1u << 16;
}  // namespace

namespace {
constexpr int kMaxPoolDevices = 64;
std::mutex g_pool_mutex;
hipMemPool_t g_pools[kMaxPoolDevices] = {};
bool g_pool_failed[kMaxPoolDevices] = {};

// The current device's pool, created at first use; null when there is none.
hipMemPool_t temp_pool() {
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess || device < 0 ||
      device >= kMaxPoolDevices) {
    (void)hipGetLastError();
    return nullptr;
  }
  std::lock_guard<std::mutex> lock(g_pool_mutex);
  if (g_pools[device] == nullptr && !g_pool_failed[device]) {
    hipMemPoolProps props = {};
    props.allocType = hipMemAllocationTypePinned;
    props.handleTypes = hipMemHandleTypeNone;
    props.location.type = hipMemLocationTypeDevice;
    props.location.id = device;
    hipMemPool_t pool = nullptr;
    if (hipMemPoolCreate(&pool, &props) == hipSuccess) {
      uint64_t keep = uint64_t{512} << 20;
      (void)hipMemPoolSetAttribute(pool, hipMemPoolAttrReleaseThreshold, &keep);
      g_pools[device] = pool;
    } else {
      (void)hipGetLastError();
      g_pool_failed[device] = true;
    }
  }
  return g_pools[device];
}
}  // namespace

hipError_t temp_malloc_async(void** ptr, size_t bytes, hipStream_t stream) {
  if (hipMemPool_t pool = temp_pool()) {
    if (hipMallocFromPoolAsync(ptr, bytes, pool, stream) == hipSuccess)
      return hipSuccess;
    (void)hipGetLastError();
  }
  return hipMallocAsync(ptr, bytes, stream);
}

void temp_free_async(void* ptr, hipStream_t stream) {
  (void)hipFreeAsync(ptr, stream);
}

KernelTimer::KernelTimer(hipStream_t stream) : stream_(stream), stop_(nullptr) {
  if (!g_timing_enabled.load(std::memory_order_relaxed)) return;
  {
    std::lock_guard<std::mutex> lock(g_timing_mutex);
    if (g_timed_kernels.size() >= kMaxTimedKernels) return;
  }
  hipEvent_t start = nullptr;
  if (hipEventCreate(&start) != hipSuccess) return;
  if (hipEventCreate(&stop_) != hipSuccess) {
    (void)hipEventDestroy(start);
    stop_ = nullptr;
    return;
  }
  (void)hipEventRecord(start, stream_);
  std::lock_guard<std::mutex> lock(g_timing_mutex);
  g_timed_kernels.emplace_back(start, stop_);
}

KernelTimer::~KernelTimer() {
  if (stop_ != nullptr) (void)hipEventRecord(stop_, stream_);
}

int report_hip_error(hipError_t err, const char* what) {
  g_last_error = std::string(hipGetErrorName(err)) + ": " +
                 hipGetErrorString(err) + " in " + what;
  return SNN_HIP_DEVICE_ERROR;
}

int report_error(int status, const std::string& text) {
  g_last_error = text;
  return status;
}

// include/portdnn/internal/conv2d/launch.h:42-97.  groups == 0 passes the
// reference's `>= 0` check and then divides by zero there; it is rejected here.
int validate(const snn_hip_conv2d_params& p) {
  SNN_REQUIRE(p.batch > 0);
  SNN_REQUIRE(p.channels > 0);
  SNN_REQUIRE(p.features > 0);
  SNN_REQUIRE(p.in_rows > 0);
  SNN_REQUIRE(p.in_cols > 0);
  SNN_REQUIRE(p.out_rows > 0);
  SNN_REQUIRE(p.out_cols > 0);
  SNN_REQUIRE(p.window_rows > 0);
  SNN_REQUIRE(p.window_cols > 0);
  SNN_REQUIRE(p.stride_rows > 0);
  SNN_REQUIRE(p.stride_cols > 0);
  SNN_REQUIRE(p.pad_rows >= 0);
  SNN_REQUIRE(p.pad_cols >= 0);
  SNN_REQUIRE(p.groups > 0);
  SNN_REQUIRE(p.channels % p.groups == 0);
  SNN_REQUIRE(p.features % p.groups == 0);
  SNN_REQUIRE(p.dilation_rows == 1);
  SNN_REQUIRE(p.dilation_cols == 1);
  // Layout combinations: NHWC goes with HWCF (0) or FHWC (2), NCHW (1) with
  // FCHW (1); INTERLEAVED (1) groups need groups > 1 and HWCF.
  SNN_REQUIRE(p.input_format == 0 || p.input_format == 1);
  SNN_REQUIRE(p.input_format != 0 ||
              (p.filter_format == 0 || p.filter_format == 2));
  SNN_REQUIRE(p.input_format != 1 || p.filter_format == 1);
  SNN_REQUIRE(p.groups != 1 || p.group_format == 0);
  SNN_REQUIRE(p.group_format != 1 || p.filter_format == 0);
  return SNN_HIP_OK;
}

// include/portdnn/internal/depthwise_conv2d/launch.h:82-112
int validate(const snn_hip_depthwise_params& p) {
  SNN_REQUIRE(p.batch > 0);
  SNN_REQUIRE(p.channels > 0);
  SNN_REQUIRE(p.channel_multiplier > 0);
  SNN_REQUIRE(p.in_rows > 0);
  SNN_REQUIRE(p.in_cols > 0);
  SNN_REQUIRE(p.out_rows > 0);
  SNN_REQUIRE(p.out_cols > 0);
  SNN_REQUIRE(p.window_rows > 0);
  SNN_REQUIRE(p.window_cols > 0);
  SNN_REQUIRE(p.stride_rows > 0);
  SNN_REQUIRE(p.stride_cols > 0);
  SNN_REQUIRE(p.pad_rows >= 0);
  SNN_REQUIRE(p.pad_cols >= 0);
  SNN_REQUIRE(p.input_format == 0);   // NHWC only
  SNN_REQUIRE(p.filter_format == 0);  // HWCF only
  return SNN_HIP_OK;
}

// include/portdnn/pooling/launch.h:56-88.  NCHW is accepted by the reference
// for Forward only; this library implements NHWC and reports NCHW as an
// invalid parameter in both directions.
int validate(const snn_hip_pooling_params& p, bool /*forward*/) {
  SNN_REQUIRE(p.batch > 0);
  SNN_REQUIRE(p.channels > 0);
  SNN_REQUIRE(p.in_rows > 0);
  SNN_REQUIRE(p.in_cols > 0);
  SNN_REQUIRE(p.out_rows > 0);
  SNN_REQUIRE(p.out_cols > 0);
  SNN_REQUIRE(p.window_rows > 0);
  SNN_REQUIRE(p.window_cols > 0);
  SNN_REQUIRE(p.stride_rows > 0);
  SNN_REQUIRE(p.stride_cols > 0);
  SNN_REQUIRE(p.pad_rows >= 0);
  SNN_REQUIRE(p.pad_cols >= 0);
  SNN_REQUIRE(p.input_format == 0);
  return SNN_HIP_OK;
}

namespace {

struct ConvSizes {
  size_t input, filter, output;
};

// include/portdnn/conv2d/sizes.h:166-179 for groups == 1.
ConvSizes conv_sizes(const snn_hip_conv2d_params& p, int direction) {
  const size_t x = static_cast<size_t>(p.batch) * p.in_rows * p.in_cols *
                   p.channels;
  const size_t w = static_cast<size_t>(p.window_rows) * p.window_cols *
                   p.channels * p.features;
  const size_t y = static_cast<size_t>(p.batch) * p.out_rows * p.out_cols *
                   p.features;
  switch (direction) {
    case SNN_HIP_FORWARD: return {x, w, y};
    case SNN_HIP_INPUT_BACKPROP: return {y, w, x};
    default: return {x, y, w};
  }
}

// The concrete selectors of include/portdnn/conv2d/selector/.
int algorithm_supports(const snn_hip_conv2d_params& p, int direction,
                       int algorithm) {
  const bool nhwc = p.input_format == 0 && p.filter_format == 0;
  switch (algorithm) {
    case SNN_HIP_ALGO_DIRECT:
    case SNN_HIP_ALGO_IM2COL:
      // constant_selector.h: always selected.
      return algorithm;
    case SNN_HIP_ALGO_TILED:
      // tiled_selector.h:45-96: Forward only, square window and stride,
      // (window, stride) in {(1,1),(1,2),(3,1),(3,2),(5,1)}.
      if (direction != SNN_HIP_FORWARD) return SNN_HIP_ALGO_NOT_SUPPORTED;
      if (p.window_rows != p.window_cols || p.stride_rows != p.stride_cols)
        return SNN_HIP_ALGO_NOT_SUPPORTED;
      if ((p.window_rows == 1 || p.window_rows == 3) &&
          (p.stride_rows == 1 || p.stride_rows == 2))
        return algorithm;
      if (p.window_rows == 5 && p.stride_rows == 1) return algorithm;
      return SNN_HIP_ALGO_NOT_SUPPORTED;
    case SNN_HIP_ALGO_WINOGRAD:
    case SNN_HIP_ALGO_WINOGRAD_LARGE:
      // winograd_selector.h:44-182.  The reference rejects a stride only when
      // BOTH strides differ from 1 (a logical AND there) and then computes a
      // stride-1 result; here both strides must be 1.
      if (p.stride_rows != 1 || p.stride_cols != 1)
        return SNN_HIP_ALGO_NOT_SUPPORTED;
      if (algorithm == SNN_HIP_ALGO_WINOGRAD &&
          ((p.window_rows == 1 && p.window_cols == 3) ||
           (p.window_rows == 3 && p.window_cols == 1)))
        return algorithm;
      if (p.window_rows == 3 && p.window_cols == 3) return algorithm;
      return SNN_HIP_ALGO_NOT_SUPPORTED;
    case SNN_HIP_ALGO_MATMUL:
      // matmul_selector.h:44-100
      if (p.stride_rows == 1 && p.stride_cols == 1 && p.window_rows == 1 &&
          p.window_cols == 1 && p.pad_rows == 0 && p.pad_cols == 0 && nhwc)
        return algorithm;
      return SNN_HIP_ALGO_NOT_SUPPORTED;
    default:
      return SNN_HIP_ALGO_NOT_SUPPORTED;
  }
}

int round_up_div(int a, int b) { return a < 0 ? 0 : (a + b - 1) / b; }

// include/portdnn/conv2d/workspace_size.h:53-76 with the kernel parameters of
// internal/conv2d/winograd/kernel_params.h:39-63 and the tile counts of
// internal/conv2d/winograd/tile_info.h:48-75.
void winograd_workspace(const snn_hip_conv2d_params& p, int direction, int m,
                        int n, int r, int s, size_t* required,
                        size_t* recommended) {
  int channels = p.channels, features = p.features;
  int out_rows = p.out_rows, out_cols = p.out_cols;
  if (direction == SNN_HIP_INPUT_BACKPROP) {
    channels = p.features;
    features = p.channels;
    out_rows = p.in_rows;
    out_cols = p.in_cols;
  }
  // Forward / input backprop tile the output in m x n blocks.  For the filter
  // gradient out <-> window are swapped and the tiles cover the swapped
  // window -- the original output extent -- in r x s blocks
  // (tile_info.h:62-73).
  const bool filbk = direction == SNN_HIP_FILTER_BACKPROP;
  const size_t a = m + r - 1, b = n + s - 1;
  const size_t tiles =
      static_cast<size_t>(round_up_div(out_rows, filbk ? r : m)) *
      round_up_div(out_cols, filbk ? s : n);
  const size_t in_t = a * b * tiles * channels;
  const size_t inter_t = a * b * tiles * features;
  const size_t fil_t = a * b * channels * features;
  *required = in_t + inter_t + fil_t;
  *recommended = static_cast<size_t>(p.batch) * (in_t + inter_t) + fil_t;
}

// include/portdnn/conv2d/workspace_size.h:100-121 with
// internal/conv2d/im2col/{tile_info.h,transform_sizes.h} for groups == 1.
void im2col_workspace(const snn_hip_conv2d_params& p, int direction,
                      size_t* required, size_t* recommended) {
  size_t tiles, tile_size, filter_t = 0;
  const size_t win = static_cast<size_t>(p.window_rows) * p.window_cols;
  if (direction == SNN_HIP_FORWARD) {
    tiles = static_cast<size_t>(p.out_rows) * p.out_cols;
    tile_size = win * p.channels;
  } else if (direction == SNN_HIP_INPUT_BACKPROP) {
    tiles = static_cast<size_t>(p.in_rows) * p.in_cols;
    tile_size = win * p.features;
    filter_t = win * p.channels * p.features;
  } else {
    tiles = win * p.channels;
    tile_size = static_cast<size_t>(p.out_rows) * p.out_cols;
  }
  const size_t in_t = tiles * tile_size;
  *required = in_t + filter_t;
  *recommended = static_cast<size_t>(p.batch) * in_t + filter_t;
}

// What a launch with `algorithm` needs.  Winograd forward / input backprop
// follow the reference's F(2x2,3x3) formula (the three-stage chain uses all of
// it, the fused kernel its transformed-filter part).  WinogradLarge runs the
// same F(2x2,3x3) / F(3x3,2x2) kernels here, so it reports their sizes, not
// the reference's F(4x4,3x3) ones.  The fused F(3x3,2x2) filter gradient keeps
// no transformed tensors, only one partial filter per slice of the tile
// range; shapes it does not take run on the implicit-GEMM kernel and need
// nothing.
//
// Half precision: every algorithm tag runs on the binary16 matrix-core kernels
// (or the direct kernel), none of which *requires* caller scratch -- without
// it they take a stream-ordered temporary -- so `required` is 0 and
// `recommended` is what the launch puts to use: the re-laid-out filter
// (forward, stride-1 input gradient) or the fp32 partial tiles / accumulation
// buffer of the filter gradient, counted in halves.
size_t f16_workspace_halves(const snn_hip_conv2d_params& p, int direction) {
  if (direction != SNN_HIP_FILTER_BACKPROP)
    return conv2d_f16_filter_pack_halves(direction, p);
  if (!conv2d_filter_backprop_f16_supports(p)) return 0;
  if (conv2d_filter_backprop_3x3_f16_supports(p))
    return 2 * conv2d_filter_backprop_3x3_f16_partial_floats(p);
  if (conv2d_filter_backprop_1x1_f16_supports(p))
    return 2 * conv2d_filter_backprop_1x1_f16_partial_floats(p);
  if (conv2d_filter_backprop_direct_f16_supports(p))
    return 2 * conv2d_filter_backprop_direct_f16_partial_floats(p);
  return 2 * static_cast<size_t>(p.window_rows) * p.window_cols * p.channels *
         p.features;
}

int workspace_size(const snn_hip_conv2d_params& p, int direction,
                   int algorithm, int dtype, size_t* required,
                   size_t* recommended) {
  *required = 0;
  *recommended = 0;
  if (dtype == SNN_HIP_DTYPE_F16) {
    if (algorithm != SNN_HIP_ALGO_DIRECT &&
        algorithm_supports(p, direction, algorithm) == algorithm)
      *recommended = f16_workspace_halves(p, direction);
    return SNN_HIP_OK;
  }
  const bool filbk = direction == SNN_HIP_FILTER_BACKPROP;
  switch (algorithm) {
    case SNN_HIP_ALGO_WINOGRAD:
    case SNN_HIP_ALGO_WINOGRAD_LARGE:
      if (!filbk && p.window_rows == 3 && p.window_cols == 3) {
        winograd_workspace(p, direction, 2, 2, 3, 3, required, recommended);
      } else if (algorithm == SNN_HIP_ALGO_WINOGRAD &&
                 conv2d_winograd_1d_supports(direction, p)) {
        // 1x3 / 3x1: F(2,3) along the window's axis, four planes
        *required = conv2d_winograd_1d_workspace(direction, p, 1);
        *recommended = conv2d_winograd_1d_workspace(direction, p, p.batch);
      } else if (filbk && conv2d_winograd_filter_backprop_supports(p)) {
        *required = conv2d_winograd_filter_backprop_workspace(p);
        *recommended = *required;
      }
      break;
    case SNN_HIP_ALGO_IM2COL:
      im2col_workspace(p, direction, required, recommended);
      break;
    default:
      break;
  }
  // The filter gradient kernel behind the Tiled / Im2col / Matmul tags
  // (channels and features in multiples of 64, or ragged shapes no other
  // matrix-core kernel fits) puts partial filters there when it is given the
  // room (else it takes a stream-ordered temporary).
  if (filbk &&
      (algorithm == SNN_HIP_ALGO_TILED || algorithm == SNN_HIP_ALGO_IM2COL ||
       algorithm == SNN_HIP_ALGO_MATMUL) &&
      algorithm_supports(p, direction, algorithm) == algorithm &&
      conv2d_filter_backprop_direct_f32_wanted(p))
    *recommended = std::max(
        *recommended, conv2d_filter_backprop_direct_f32_partial_floats(p));
  return SNN_HIP_OK;
}

// Device policy standing in for get_default_selector
// (src/conv2d/selector/default_selector.cc:49-128): 1x1 stride-1 unpadded
// convolutions are one GEMM; everything else is the implicit-GEMM path, which
// the Im2col tag names (Tiled where the reference's TiledSelector accepts it).
// Half precision has no Winograd kernels: its 3x3 layers run on the LDS-tile
// kernel behind the Tiled / Im2col tags, so the policy never answers Winograd
// for it (a Winograd tag would still run, on those same kernels).
int default_algorithm(const snn_hip_conv2d_params& p, int direction,
                      int dtype) {
  if (algorithm_supports(p, direction, SNN_HIP_ALGO_MATMUL))
    return SNN_HIP_ALGO_MATMUL;
  if (dtype == SNN_HIP_DTYPE_F16)
    return algorithm_supports(p, direction, SNN_HIP_ALGO_TILED)
               ? SNN_HIP_ALGO_TILED
               : SNN_HIP_ALGO_IM2COL;
  // 3x3 stride-1 layers whose channel counts fit the fused Winograd kernel:
  // measured 1.3-1.5x faster than the implicit GEMM on the batch-32 ResNet
  // shapes.  The caller sizes the workspace with query_workspace_size for
  // the same selector, as for any Winograd launch.
  if (algorithm_supports(p, direction, SNN_HIP_ALGO_WINOGRAD) &&
      conv2d_winograd_fused_supports(direction, p) &&
      static_cast<long long>(p.batch) * p.out_rows * p.out_cols >= 1024)
    return SNN_HIP_ALGO_WINOGRAD;
  // The fused F(3x3,2x2) filter gradient: measured 1.2-1.6x faster than the
  // implicit GEMM on the batch-32 ResNet shapes once the tile range gives
  // every work-group a few steps.
  if (direction == SNN_HIP_FILTER_BACKPROP &&
      algorithm_supports(p, direction, SNN_HIP_ALGO_WINOGRAD) &&
      conv2d_winograd_filter_backprop_supports(p) && p.channels % 32 == 0 &&
      p.features % 32 == 0 &&
      static_cast<long long>(p.batch) * p.out_rows * p.out_cols >= 1024)
    return SNN_HIP_ALGO_WINOGRAD;
  if (algorithm_supports(p, direction, SNN_HIP_ALGO_TILED))
    return SNN_HIP_ALGO_TILED;
  return SNN_HIP_ALGO_IM2COL;
}

inline bool aligned16(const void* p) {
  return (reinterpret_cast<uintptr_t>(p) & 15u) == 0;
}

// Tiled / Im2col / Matmul: the MFMA implicit-GEMM kernel wherever its vector
// width and alignment requirements hold, the direct kernel otherwise.
template <typename T>
int launch_gemm_path(int direction, const T* input, const T* filter, T* output,
                     const snn_hip_conv2d_params& p, hipStream_t s,
                     T* workspace = nullptr, size_t workspace_elems = 0,
                     const LaunchOptions* epilogue = nullptr);

// out[r][j] = j < valid ? in[r][j] : 0 for j < out_cols: widens (zeros in the
// new columns) or narrows the last dimension of a row-major matrix.
template <typename T>
__global__ void __launch_bounds__(256)
    copy_columns_kernel(const T* __restrict__ in, int in_cols,
                        T* __restrict__ out, int out_cols, int valid,
                        size_t total) {
  const size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
  if (i >= total) return;
  const size_t r = i / out_cols;
  const int j = static_cast<int>(i - r * out_cols);
  out[i] = j < valid ? in[r * in_cols + j] : static_cast<T>(0);
}

template <typename T>
void copy_columns(const T* in, int in_cols, T* out, int out_cols, int valid,
                  size_t rows, hipStream_t s) {
  const size_t total = rows * out_cols;
  hipLaunchKernelGGL(copy_columns_kernel<T>,
                     dim3(static_cast<unsigned>(ceil_div(total, size_t{256}))),
                     dim3(256), 0, s, in, in_cols, out, out_cols, valid, total);
}

// Feature counts that are not multiples of 4 (an RGB output layer, 21
// classes): the matrix-core kernels load and store features four at a time,
// so for a forward convolution or an input gradient the tensors that carry
// the feature dimension are copied into stream-ordered temporaries with the
// count rounded up (zeros in the new columns), the launch runs on the padded
// problem -- when `padded_ok` says a matrix-core kernel takes it -- and a
// forward result is copied back without the padding.  The copies move a
// fraction of what the one-lane-per-output kernel would otherwise read.
// Returns -1 when it does not apply.
template <typename T, typename Supports>
int launch_gemm_path_padded(int direction, const T* input, const T* filter,
                            T* output, const snn_hip_conv2d_params& p,
                            hipStream_t s, const LaunchOptions* epilogue,
                            Supports padded_ok) {
  if (direction == SNN_HIP_FILTER_BACKPROP || p.features % 4 == 0) return -1;
  if (epilogue != nullptr && epilogue->wanted()) return -1;  // bias has K entries
  // (an input gradient over three features or fewer is a short loop per
  // output: the direct kernel measured faster, 80 against 99 us)
  if (direction == SNN_HIP_INPUT_BACKPROP && p.features < 4) return -1;
  snn_hip_conv2d_params q = p;
  q.features = (p.features + 3) / 4 * 4;
  if (!padded_ok(q)) return -1;
  const size_t pixels = static_cast<size_t>(p.batch) * p.out_rows * p.out_cols;
  const size_t filter_rows =
      static_cast<size_t>(p.window_rows) * p.window_cols * p.channels;
  // (small problems stay where they were: three more launches and two
  // temporaries cost more than the direct kernel's whole run)
  if (pixels * filter_rows * p.features < (size_t{1} << 24)) return -1;
  // one temporary holds both copies (the filter's rounded up to 256 bytes)
  const size_t filter_elems =
      (filter_rows * q.features + 127) / 128 * 128;
  void* wide_filter = nullptr;
  // (no room for the copies: the launch stays on the path it had)
  if (temp_malloc_async(&wide_filter,
                        (filter_elems + pixels * q.features) * sizeof(T),
                        s) != hipSuccess) {
    (void)hipGetLastError();
    return -1;
  }
  void* const wide_pixels = static_cast<T*>(wide_filter) + filter_elems;
  copy_columns(filter, p.features, static_cast<T*>(wide_filter), q.features,
               p.features, filter_rows, s);
  int status;
  if (direction == SNN_HIP_FORWARD) {
    status = launch_gemm_path<T>(direction, input, static_cast<T*>(wide_filter),
                                 static_cast<T*>(wide_pixels), q, s, nullptr, 0,
                                 epilogue);
    copy_columns(static_cast<const T*>(wide_pixels), q.features, output,
                 p.features, p.features, pixels, s);
  } else {
    copy_columns(input, p.features, static_cast<T*>(wide_pixels), q.features,
                 p.features, pixels, s);
    status = launch_gemm_path<T>(direction, static_cast<T*>(wide_pixels),
                                 static_cast<T*>(wide_filter), output, q, s,
                                 nullptr, 0, epilogue);
  }
  const hipError_t err = hipGetLastError();
  temp_free_async(wide_filter, s);
  if (status != SNN_HIP_OK) return status;
  if (err != hipSuccess) return report_hip_error(err, "padded features");
  return SNN_HIP_OK;
}
template <>
int launch_gemm_path<float>(int direction, const float* input,
                            const float* filter, float* output,
                            const snn_hip_conv2d_params& p, hipStream_t s,
                            float* workspace, size_t workspace_elems,
                            const LaunchOptions* epilogue);

template <typename From, typename To>
__global__ void __launch_bounds__(256)
    convert_kernel(const From* __restrict__ in, To* __restrict__ out, size_t n) {
  const size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
  if (i < n) out[i] = static_cast<To>(in[i]);
}

// Four elements per lane.
template <typename From, typename To>
__global__ void __launch_bounds__(256)
    convert4_kernel(const From* __restrict__ in, To* __restrict__ out,
                    size_t n_vec) {
  typedef From from4 __attribute__((ext_vector_type(4)));
  typedef To to4 __attribute__((ext_vector_type(4)));
  const size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
  if (i >= n_vec) return;
  const from4 v = reinterpret_cast<const from4*>(in)[i];
  to4 r;
#pragma unroll
  for (int e = 0; e < 4; ++e) r[e] = static_cast<To>(v[e]);
  reinterpret_cast<to4*>(out)[i] = r;
}

template <typename From, typename To>
void convert(const From* in, To* out, size_t n, hipStream_t s) {
  const bool vec = n % 4 == 0 &&
                   (reinterpret_cast<uintptr_t>(in) % (4 * sizeof(From))) == 0 &&
                   (reinterpret_cast<uintptr_t>(out) % (4 * sizeof(To))) == 0;
  if (vec)
    hipLaunchKernelGGL((convert4_kernel<From, To>),
                       dim3(static_cast<unsigned>(ceil_div(n / 4, size_t{256}))),
                       dim3(256), 0, s, in, out, n / 4);
  else
    hipLaunchKernelGGL((convert_kernel<From, To>),
                       dim3(static_cast<unsigned>(ceil_div(n, size_t{256}))),
                       dim3(256), 0, s, in, out, n);
}

// A binary16 launch that no binary16 matrix-core kernel takes (three input
// channels, channel or feature counts that are not multiples of 4, strided
// input gradients) through the fp32 kernels: operands widened into
// stream-ordered temporaries, the fp32 launch -- every path it has -- and the
// result rounded back.  Products and sums are then fp32 on binary16-rounded
// operands, as in the binary16 kernels.  From 2^24 multiply-adds; returns -1
// when it does not apply.
int launch_f16_through_fp32(int direction, const _Float16* input,
                            const _Float16* filter, _Float16* output,
                            const snn_hip_conv2d_params& p, hipStream_t s) {
  const double macs = static_cast<double>(p.batch) * p.out_rows * p.out_cols *
                      p.window_rows * p.window_cols * p.channels * p.features;
  if (macs < double(1 << 24)) return -1;
  const ConvSizes sz = conv_sizes(p, direction);
  // The 7x7 stride-2 three-channel stem, forward: the fp32 kernel rounds its
  // output -- the large tensor -- to binary16 on the store, so only the image
  // and the filter are widened (430 -> 328 us at batch 128).  (The filter
  // gradient reading dY as binary16, one 2-byte load per lane where the fp32
  // kernel has a 4-byte one, measured slower than the widening pass it saves:
  // 623 against 444 us.)
  if (direction == SNN_HIP_FORWARD && conv2d_stem_supports(p) &&
      (reinterpret_cast<uintptr_t>(output) & 7u) == 0) {
    auto padded = [](size_t floats) { return (floats + 63) / 64 * 64; };
    void* block = nullptr;
    if (temp_malloc_async(&block,
                          (padded(sz.input) + padded(sz.filter)) * sizeof(float),
                          s) == hipSuccess) {
      float* const in32 = static_cast<float*>(block);
      float* const fil32 = in32 + padded(sz.input);
      convert(input, in32, sz.input, s);
      convert(filter, fil32, sz.filter, s);
      const int status =
          launch_conv2d_stem_f32_to_f16(in32, fil32, output, p, s);
      const hipError_t err = hipGetLastError();
      temp_free_async(block, s);
      if (status != SNN_HIP_OK) return status;
      if (err != hipSuccess) return report_hip_error(err, "binary16 stem");
      return SNN_HIP_OK;
    }
    (void)hipGetLastError();
  }
  // One stream-ordered temporary for the three widened tensors and the
  // workspace the fp32 launch would otherwise allocate for itself (every
  // allocation costs tens of microseconds of host time).
  auto padded = [](size_t floats) { return (floats + 63) / 64 * 64; };
  size_t ws_required = 0, ws_floats = 0;
  (void)workspace_size(p, direction, SNN_HIP_ALGO_IM2COL, SNN_HIP_DTYPE_F32,
                       &ws_required, &ws_floats);
  if (ws_floats > (size_t{256} << 20) / sizeof(float)) ws_floats = 0;
  const size_t total = padded(sz.input) + padded(sz.filter) +
                       padded(sz.output) + padded(ws_floats);
  void* block = nullptr;
  if (temp_malloc_async(&block, total * sizeof(float), s) != hipSuccess) {
    // (no room for the copies: the launch stays on the path it had)
    (void)hipGetLastError();
    return -1;
  }
  float* const in32 = static_cast<float*>(block);
  float* const fil32 = in32 + padded(sz.input);
  float* const out32 = fil32 + padded(sz.filter);
  float* const ws32 = ws_floats != 0 ? out32 + padded(sz.output) : nullptr;
  convert(input, in32, sz.input, s);
  convert(filter, fil32, sz.filter, s);
  const int status = launch_gemm_path<float>(direction, in32, fil32, out32, p,
                                             s, ws32, ws_floats, nullptr);
  if (status == SNN_HIP_OK)
    convert(static_cast<const float*>(out32), output, sz.output, s);
  const hipError_t err = hipGetLastError();
  temp_free_async(block, s);
  if (status != SNN_HIP_OK) return status;
  if (err != hipSuccess) return report_hip_error(err, "binary16 through fp32");
  return SNN_HIP_OK;
}

template <>
int launch_gemm_path<_Float16>(int direction, const _Float16* input,
                               const _Float16* filter, _Float16* output,
                               const snn_hip_conv2d_params& p, hipStream_t s,
                               _Float16* workspace, size_t workspace_elems,
                               const LaunchOptions*) {
  // (a gradient of at most eight channels: the binary16 kernels' 64-channel
  // tiles would be nearly empty, fp32 has kernels for such layers -- 224x224
  // 3 <- 64, 3x3, at batch 8: 286 us on the general binary16 kernel over a
  // copy widened to four channels, 69 us in fp32)
  if (direction == SNN_HIP_INPUT_BACKPROP && p.channels <= 8) {
    const int rc = launch_f16_through_fp32(direction, input, filter, output, p, s);
    if (rc >= 0) return rc;
  }
  if (direction == SNN_HIP_INPUT_BACKPROP && aligned16(output)) {
    const int padded = launch_gemm_path_padded<_Float16>(
        direction, input, filter, output, p, s, nullptr,
        [](const snn_hip_conv2d_params& q) {
          return conv2d_input_backprop_f16_supports(q) ||
                 conv2d_input_backprop_general_f16_supports(q);
        });
    if (padded >= 0) return padded;
  }
  if (direction == SNN_HIP_FORWARD && conv2d_igemm_f16_supports(p) &&
      aligned16(input) && aligned16(filter) && aligned16(output))
    return launch_conv2d_igemm_f16(input, filter, output, p, workspace,
                                   workspace_elems, s);
  if (direction == SNN_HIP_FORWARD &&
      conv2d_forward_general_f16_supports(p) && aligned16(input) &&
      aligned16(filter) && aligned16(output))
    return launch_conv2d_forward_general_f16(input, filter, output, p, s);
  if (direction == SNN_HIP_INPUT_BACKPROP &&
      conv2d_input_backprop_f16_supports(p) && aligned16(input) &&
      aligned16(filter) && aligned16(output))
    return launch_conv2d_input_backprop_f16(input, filter, output, p,
                                            workspace, workspace_elems, s);
  // (a strided input gradient from 2^30 multiply-adds: the fp32 launch splits
  // it into stride classes, the general binary16 kernel multiplies the zeros
  // of the taps that do not reach a pixel -- 1.39 ms against 67 us forward for
  // 56x56x128 -> 128, 3x3 stride 2, at batch 128)
  if (direction == SNN_HIP_INPUT_BACKPROP &&
      conv2d_strided_input_backprop_f16_supports(p) && aligned16(input) &&
      aligned16(filter) && aligned16(output)) {
    const int rc =
        launch_conv2d_strided_input_backprop_f16(input, filter, output, p, s);
    if (rc >= 0) return rc;
  }
  if (direction == SNN_HIP_INPUT_BACKPROP &&
      (p.stride_rows > 1 || p.stride_cols > 1) &&
      static_cast<double>(p.batch) * p.out_rows * p.out_cols * p.window_rows *
              p.window_cols * p.channels * p.features >= double(1 << 30)) {
    const int rc = launch_f16_through_fp32(direction, input, filter, output, p, s);
    if (rc >= 0) return rc;
  }
  if (direction == SNN_HIP_INPUT_BACKPROP &&
      conv2d_input_backprop_general_f16_supports(p) && aligned16(input) &&
      aligned16(filter))
    return launch_conv2d_input_backprop_general_f16(input, filter, output, p,
                                                    s);
  // (few (tap, channel) pairs -- a three-channel stem: fp32 has kernels built
  // for that; 64-channel tiles would be nearly empty)
  if (direction == SNN_HIP_FILTER_BACKPROP && p.channels <= 8 &&
      p.window_rows * p.window_cols * p.channels <= 768) {
    const int rc = launch_f16_through_fp32(direction, input, filter, output, p, s);
    if (rc >= 0) return rc;
  }
  if (direction == SNN_HIP_FILTER_BACKPROP &&
      conv2d_filter_backprop_f16_supports(p) && aligned16(input) &&
      aligned16(filter))
    return launch_conv2d_filter_backprop_f16(input, filter, output, p,
                                             workspace, workspace_elems, s);
  {
    const int rc = launch_f16_through_fp32(direction, input, filter, output, p, s);
    if (rc >= 0) return rc;
  }
  return launch_conv2d_direct<_Float16>(direction, input, filter, output, p, s);
}
template <>
int launch_gemm_path<float>(int direction, const float* input,
                            const float* filter, float* output,
                            const snn_hip_conv2d_params& p, hipStream_t s,
                            float* workspace, size_t workspace_elems,
                            const LaunchOptions* epilogue) {
  // The implicit-GEMM filter gradient meets its partial tiles through float
  // atomics; a launch that must be reproducible takes the direct kernel (one
  // lane per filter element, fixed order) instead.  The kernel for channels
  // and features in multiples of 64 adds in a fixed order and serves both.
  const bool atomics_only = direction == SNN_HIP_FILTER_BACKPROP &&
                            epilogue != nullptr && epilogue->deterministic &&
                            !conv2d_filter_backprop_direct_f32_wanted(p, true);
  if ((direction == SNN_HIP_FORWARD && aligned16(input)) ||
      (direction == SNN_HIP_INPUT_BACKPROP && aligned16(output))) {
    const int padded = launch_gemm_path_padded<float>(
        direction, input, filter, output, p, s, epilogue,
        [direction](const snn_hip_conv2d_params& q) {
          return conv2d_igemm_supports(direction, q);
        });
    if (padded >= 0) return padded;
  }
  if (conv2d_igemm_supports(direction, p) && aligned16(input) &&
      aligned16(filter) && aligned16(output) && !atomics_only)
    return launch_conv2d_igemm_f32(direction, input, filter, output, p, s,
                                   workspace, workspace_elems, epilogue);
  return launch_conv2d_direct<float>(direction, input, filter, output, p, s);
}

// Winograd / WinogradLarge: F(2x2,3x3) for forward and input backprop of 3x3
// stride-1 convolutions and F(3x3,2x2) for their filter gradient; F(2,3)
// along the window's axis for the 1x3 / 3x1 windows the selector also accepts
// (forward and input backprop; their filter gradient, a reduction over every
// tile with 3 results per (channel, feature), gains nothing over the implicit
// GEMM and runs there, as do shapes the Winograd kernels do not take).
// WinogradLarge runs the same kernels as Winograd, because the larger
// constants of F(4x4,3x3) cost accuracy against the fp32 bar.
template <typename T>
int launch_winograd_path(int direction, const T* input, const T* filter,
                         T* output, const snn_hip_conv2d_params& p,
                         T* workspace, size_t workspace_elems, hipStream_t s,
                         const LaunchOptions* epilogue = nullptr) {
  return launch_gemm_path<T>(direction, input, filter, output, p, s, workspace,
                             workspace_elems);
}
template <>
int launch_winograd_path<float>(int direction, const float* input,
                                const float* filter, float* output,
                                const snn_hip_conv2d_params& p,
                                float* workspace, size_t workspace_elems,
                                hipStream_t s, const LaunchOptions* epilogue) {
  // SNN_HIP_WINO_UNFUSED is a development switch that forces the three-stage
  // chain on shapes the fused kernel would take.
  // (the input gradient's filter transform reads the filter 16 bytes at a time)
  if (conv2d_winograd_fused_supports(direction, p) && aligned16(input) &&
      aligned16(output) && aligned16(workspace) &&
      (direction != SNN_HIP_INPUT_BACKPROP || aligned16(filter)) &&
      SNN_TUNING_ENV("SNN_HIP_WINO_UNFUSED") == nullptr)
    return launch_conv2d_winograd_fused_f32(direction, input, filter, output,
                                            p, workspace, workspace_elems, s,
                                            epilogue);
  if (conv2d_winograd_supports(direction, p))
    return launch_conv2d_winograd_f32(
        direction, input, filter, output, p, workspace, workspace_elems, s,
        epilogue != nullptr && epilogue->deterministic);
  if (conv2d_winograd_1d_supports(direction, p) && aligned16(workspace))
    return launch_conv2d_winograd_1d_f32(
        direction, input, filter, output, p, workspace, workspace_elems, s,
        epilogue != nullptr && epilogue->deterministic);
  if (direction == SNN_HIP_FILTER_BACKPROP &&
      conv2d_winograd_filter_backprop_supports(p) && aligned16(input) &&
      aligned16(filter) && aligned16(output) && aligned16(workspace))
    return launch_conv2d_winograd_filter_backprop_f32(
        input, filter, output, p, workspace, workspace_elems, s);
  return launch_gemm_path<float>(direction, input, filter, output, p, s,
                                 nullptr, 0, epilogue);
}

template <typename T>
int conv2d_dispatch(int direction, const T* input, const T* filter, T* output,
                    const snn_hip_conv2d_params* params, int algorithm,
                    T* workspace, size_t workspace_elems, void* stream,
                    const LaunchOptions* epilogue = nullptr);

// NCHW activations with an FCHW filter (the only filter layout portDNN
// accepts with NCHW, include/portdnn/internal/conv2d/launch.h:86-88): the
// operands are rewritten as NHWC / HWCF into stream-ordered temporaries, the
// convolution runs on them and the result is written back in the caller's
// layout.  Only fp32.
template <typename T>
int conv2d_nchw(int, const T*, const T*, T*, const snn_hip_conv2d_params&,
                int, hipStream_t) {
  return SNN_HIP_INVALID_ALGORITHM;
}
template <>
int conv2d_nchw<float>(int direction, const float* input, const float* filter,
                       float* output, const snn_hip_conv2d_params& p,
                       int algorithm, hipStream_t s) {
  const ConvSizes sz = conv_sizes(p, direction);
  const int taps = p.window_rows * p.window_cols;
  const int in_hw = p.in_rows * p.in_cols, out_hw = p.out_rows * p.out_cols;
  float* tmp = nullptr;
  if (temp_malloc_async(reinterpret_cast<void**>(&tmp),
                     (sz.input + sz.filter + sz.output) * sizeof(float), s) !=
      hipSuccess)
    return SNN_HIP_ALLOCATION_PROBLEM;
  float* t_in = tmp;
  float* t_fil = tmp + sz.input;
  float* t_out = t_fil + sz.filter;
  // operand roles per direction (include/snn_hip.h): tensor shapes as
  // (batches, channels, pixels) for the activations
  struct Act { int c, hw; };
  const Act x{p.channels, in_hw}, y{p.features, out_hw};
  const Act in_a = direction == SNN_HIP_INPUT_BACKPROP ? y : x;
  const bool fil_is_filter = direction != SNN_HIP_FILTER_BACKPROP;
  const Act out_a = direction == SNN_HIP_FORWARD ? y : x;
  int rc = launch_transpose_batched_f32(input, t_in, p.batch, in_a.c, in_a.hw,
                                        s);
  if (rc == SNN_HIP_OK)
    rc = fil_is_filter
             ? launch_permute_filter_f32(filter, t_fil, p.features, p.channels,
                                         taps, true, s)
             : launch_transpose_batched_f32(filter, t_fil, p.batch, y.c, y.hw,
                                            s);
  if (rc == SNN_HIP_OK) {
    snn_hip_conv2d_params q = p;
    q.input_format = 0;
    q.filter_format = 0;
    rc = conv2d_dispatch<float>(direction, t_in, t_fil, t_out, &q, algorithm,
                                nullptr, 0, s);
  }
  if (rc == SNN_HIP_OK)
    rc = direction == SNN_HIP_FILTER_BACKPROP
             ? launch_permute_filter_f32(t_out, output, p.features, p.channels,
                                         taps, false, s)
             : launch_transpose_batched_f32(t_out, output, p.batch, out_a.hw,
                                            out_a.c, s);
  temp_free_async(tmp, s);
  return rc;
}

template <typename T>
int conv2d_dispatch(int direction, const T* input, const T* filter, T* output,
                    const snn_hip_conv2d_params* params, int algorithm,
                    T* workspace, size_t workspace_elems, void* stream,
                    const LaunchOptions* epilogue) {
  if (params == nullptr) return SNN_HIP_INVALID_PARAMETER;
  const snn_hip_conv2d_params& p = *params;
  const int v = validate(p);
  if (v != SNN_HIP_OK) return v;
  if (input == nullptr || filter == nullptr || output == nullptr)
    return SNN_HIP_INVALID_PARAMETER;
  // Grouped and FHWC convolutions are outside this library.
  if (p.groups != 1 || p.filter_format == 2) return SNN_HIP_INVALID_ALGORITHM;
  // include/portdnn/internal/conv2d/launch.h:81-88: NHWC goes with HWCF,
  // NCHW with FCHW.
  if ((p.input_format == 0) != (p.filter_format == 0))
    return SNN_HIP_INVALID_PARAMETER;
  if (algorithm_supports(p, direction, algorithm) == SNN_HIP_ALGO_NOT_SUPPORTED)
    return SNN_HIP_INVALID_ALGORITHM;
  const ConvSizes sz = conv_sizes(p, direction);
  if (!fits_int32(sz.input) || !fits_int32(sz.filter) || !fits_int32(sz.output))
    return SNN_HIP_INDEX_EXCEEDED;
  hipStream_t s = as_stream(stream);
  if (p.input_format != 0) {
    // include/portdnn/internal/conv2d/launch.h:191-194: NCHW is served by the
    // Direct algorithm only.
    if (algorithm != SNN_HIP_ALGO_DIRECT) return SNN_HIP_INVALID_ALGORITHM;
    if (epilogue != nullptr && epilogue->wanted())
      return SNN_HIP_INVALID_ALGORITHM;  // bias is indexed by the last dim
    return conv2d_nchw<T>(direction, input, filter, output, p, algorithm, s);
  }
  switch (algorithm) {
    case SNN_HIP_ALGO_WINOGRAD:
    case SNN_HIP_ALGO_WINOGRAD_LARGE: {
      // internal/conv2d/winograd/launch.h:271-286: a Winograd launch without
      // the workspace its transforms need reports InsufficientWorkspace.
      size_t required = 0, recommended = 0;
      workspace_size(p, direction, algorithm,
                     std::is_same<T, float>::value ? SNN_HIP_DTYPE_F32
                                                   : SNN_HIP_DTYPE_F16,
                     &required, &recommended);
      if (required > 0 && (workspace == nullptr || workspace_elems < required))
        return SNN_HIP_INSUFFICIENT_WORKSPACE;
      return launch_winograd_path<T>(direction, input, filter, output, p,
                                     workspace, workspace_elems, s, epilogue);
    }
    case SNN_HIP_ALGO_TILED:
    case SNN_HIP_ALGO_IM2COL:
    case SNN_HIP_ALGO_MATMUL:
      return launch_gemm_path<T>(direction, input, filter, output, p, s,
                                 workspace, workspace_elems, epilogue);
    default:
      return launch_conv2d_direct<T>(direction, input, filter, output, p, s);
  }
}

template <typename T>
int depthwise_dispatch(int direction, const T* input, const T* filter,
                       T* output, const snn_hip_depthwise_params* params,
                       void* stream) {
  if (params == nullptr) return SNN_HIP_INVALID_PARAMETER;
  const int v = validate(*params);
  if (v != SNN_HIP_OK) return v;
  if (input == nullptr || filter == nullptr || output == nullptr)
    return SNN_HIP_INVALID_PARAMETER;
  const snn_hip_depthwise_params& p = *params;
  const size_t cm = static_cast<size_t>(p.channels) * p.channel_multiplier;
  if (!fits_int32(static_cast<size_t>(p.batch) * p.in_rows * p.in_cols *
                  p.channels) ||
      !fits_int32(static_cast<size_t>(p.batch) * p.out_rows * p.out_cols * cm))
    return SNN_HIP_INDEX_EXCEEDED;
  return launch_depthwise<T>(direction, input, filter, output, p,
                             as_stream(stream));
}

int pooling_check(const snn_hip_pooling_params* params, bool forward) {
  if (params == nullptr) return SNN_HIP_INVALID_PARAMETER;
  const int v = validate(*params, forward);
  if (v != SNN_HIP_OK) return v;
  const snn_hip_pooling_params& p = *params;
  if (!fits_int32(static_cast<size_t>(p.batch) * p.in_rows * p.in_cols *
                  p.channels) ||
      !fits_int32(static_cast<size_t>(p.batch) * p.out_rows * p.out_cols *
                  p.channels))
    return SNN_HIP_INDEX_EXCEEDED;
  return SNN_HIP_OK;
}

}  // namespace
}  // namespace snn

using namespace snn;

extern "C" {

int snn_hip_version(void) { return 100; }  // 0.1.0

const char* snn_hip_status_string(int status) {
  switch (status) {
    case SNN_HIP_OK: return "OK";
    case SNN_HIP_INVALID_ALGORITHM: return "InvalidAlgorithm";
    case SNN_HIP_INDEX_EXCEEDED: return "IndexExceeded";
    case SNN_HIP_INSUFFICIENT_WORKSPACE: return "InsufficientWorkspace";
    case SNN_HIP_ALLOCATION_PROBLEM: return "AllocationProblem";
    case SNN_HIP_INVALID_PARAMETER: return "InvalidParameter";
    case SNN_HIP_DEVICE_ERROR: return "DeviceError";
    default: return "Unknown";
  }
}

const char* snn_hip_last_error(void) { return g_last_error.c_str(); }

int snn_hip_kernel_timing_enable(int enable) {
  snn::g_timing_enabled.store(enable != 0);
  return SNN_HIP_OK;
}

int snn_hip_kernel_timing_read(double* total_ms, int* kernels) {
  if (total_ms == nullptr || kernels == nullptr)
    return SNN_HIP_INVALID_PARAMETER;
  double sum = 0.0;
  int n = 0;
  int status = SNN_HIP_OK;
  std::vector<std::pair<hipEvent_t, hipEvent_t>> pairs;
  {
    std::lock_guard<std::mutex> lock(snn::g_timing_mutex);
    pairs.swap(snn::g_timed_kernels);
  }
  for (auto& pair : pairs) {
    float ms = 0.f;
    hipError_t err = hipEventSynchronize(pair.second);
    if (err == hipSuccess)
      err = hipEventElapsedTime(&ms, pair.first, pair.second);
    if (err == hipSuccess) {
      sum += ms;
      ++n;
    } else {
      status = snn::report_hip_error(err, "kernel timing");
    }
    (void)hipEventDestroy(pair.first);
    (void)hipEventDestroy(pair.second);
  }
  *total_ms = sum;
  *kernels = n;
  return status;
}

int snn_hip_temporary_memory_stats(unsigned long long* reserved_bytes,
                                   unsigned long long* used_high_bytes,
                                   int reset_high) {
  if (reserved_bytes == nullptr || used_high_bytes == nullptr)
    return SNN_HIP_INVALID_PARAMETER;
  *reserved_bytes = 0;
  *used_high_bytes = 0;
  int device = 0;
  hipError_t err = hipGetDevice(&device);
  if (err != hipSuccess) return snn::report_hip_error(err, "hipGetDevice");
  hipMemPool_t pools[2] = {nullptr, nullptr};
  if (device >= 0 && device < snn::kMaxPoolDevices) {
    std::lock_guard<std::mutex> lock(snn::g_pool_mutex);
    pools[0] = snn::g_pools[device];
  }
  if (hipDeviceGetDefaultMemPool(&pools[1], device) != hipSuccess) {
    (void)hipGetLastError();
    pools[1] = nullptr;
  }
  for (hipMemPool_t pool : pools) {
    if (pool == nullptr) continue;
    uint64_t reserved = 0, high = 0;
    err = hipMemPoolGetAttribute(pool, hipMemPoolAttrReservedMemCurrent,
                                 &reserved);
    if (err == hipSuccess)
      err = hipMemPoolGetAttribute(pool, hipMemPoolAttrUsedMemHigh, &high);
    if (err != hipSuccess)
      return snn::report_hip_error(err, "hipMemPoolGetAttribute");
    *reserved_bytes += reserved;
    *used_high_bytes += high;
    if (reset_high != 0) {
      uint64_t zero = 0;
      (void)hipMemPoolSetAttribute(pool, hipMemPoolAttrUsedMemHigh, &zero);
    }
  }
  return SNN_HIP_OK;
}

int snn_hip_conv2d_forward_f32(const float* input, const float* filter,
                               float* output,
                               const snn_hip_conv2d_params* params,
                               int algorithm, float* workspace,
                               size_t workspace_elems, void* stream) {
  return conv2d_dispatch<float>(SNN_HIP_FORWARD, input, filter, output, params,
                                algorithm, workspace, workspace_elems, stream);
}

int snn_hip_conv2d_input_backprop_f32(const float* input, const float* filter,
                                      float* output,
                                      const snn_hip_conv2d_params* params,
                                      int algorithm, float* workspace,
                                      size_t workspace_elems, void* stream) {
  return conv2d_dispatch<float>(SNN_HIP_INPUT_BACKPROP, input, filter, output,
                                params, algorithm, workspace, workspace_elems,
                                stream);
}

int snn_hip_conv2d_filter_backprop_f32(const float* input, const float* filter,
                                       float* output,
                                       const snn_hip_conv2d_params* params,
                                       int algorithm, float* workspace,
                                       size_t workspace_elems, void* stream) {
  return conv2d_dispatch<float>(SNN_HIP_FILTER_BACKPROP, input, filter, output,
                                params, algorithm, workspace, workspace_elems,
                                stream);
}

int snn_hip_conv2d_forward_f16(const void* input, const void* filter,
                               void* output,
                               const snn_hip_conv2d_params* params,
                               int algorithm, void* workspace,
                               size_t workspace_elems, void* stream) {
  return conv2d_dispatch<_Float16>(
      SNN_HIP_FORWARD, static_cast<const _Float16*>(input),
      static_cast<const _Float16*>(filter), static_cast<_Float16*>(output),
      params, algorithm, static_cast<_Float16*>(workspace), workspace_elems,
      stream);
}

int snn_hip_conv2d_input_backprop_f16(const void* input, const void* filter,
                                      void* output,
                                      const snn_hip_conv2d_params* params,
                                      int algorithm, void* workspace,
                                      size_t workspace_elems, void* stream) {
  return conv2d_dispatch<_Float16>(
      SNN_HIP_INPUT_BACKPROP, static_cast<const _Float16*>(input),
      static_cast<const _Float16*>(filter), static_cast<_Float16*>(output),
      params, algorithm, static_cast<_Float16*>(workspace), workspace_elems,
      stream);
}

int snn_hip_conv2d_filter_backprop_f16(const void* input, const void* filter,
                                       void* output,
                                       const snn_hip_conv2d_params* params,
                                       int algorithm, void* workspace,
                                       size_t workspace_elems, void* stream) {
  return conv2d_dispatch<_Float16>(
      SNN_HIP_FILTER_BACKPROP, static_cast<const _Float16*>(input),
      static_cast<const _Float16*>(filter), static_cast<_Float16*>(output),
      params, algorithm, static_cast<_Float16*>(workspace), workspace_elems,
      stream);
}

int snn_hip_conv2d_deterministic_f32(int direction, const float* input,
                                     const float* filter, float* output,
                                     const snn_hip_conv2d_params* params,
                                     int algorithm, float* workspace,
                                     size_t workspace_elems, void* stream) {
  if (direction < SNN_HIP_FORWARD || direction > SNN_HIP_FILTER_BACKPROP)
    return SNN_HIP_INVALID_PARAMETER;
  LaunchOptions options;
  options.deterministic = true;
  return conv2d_dispatch<float>(direction, input, filter, output, params,
                                algorithm, workspace, workspace_elems, stream,
                                &options);
}

int snn_hip_conv2d_prepare_filter_f32(int direction, const float* filter,
                                      const snn_hip_conv2d_params* params,
                                      int algorithm, float* workspace,
                                      size_t workspace_elems, void* stream) {
  if (params == nullptr || filter == nullptr)
    return SNN_HIP_INVALID_PARAMETER;
  if (direction < SNN_HIP_FORWARD || direction > SNN_HIP_FILTER_BACKPROP)
    return SNN_HIP_INVALID_PARAMETER;
  const snn_hip_conv2d_params& p = *params;
  const int v = validate(p);
  if (v != SNN_HIP_OK) return v;
  if (p.groups != 1 || p.filter_format == 2) return SNN_HIP_INVALID_ALGORITHM;
  if (algorithm_supports(p, direction, algorithm) == SNN_HIP_ALGO_NOT_SUPPORTED)
    return SNN_HIP_INVALID_ALGORITHM;
  // Only the fused Winograd forward / input-gradient kernels keep anything
  // derived from the filter alone; every other path has nothing to prepare.
  if ((algorithm != SNN_HIP_ALGO_WINOGRAD &&
       algorithm != SNN_HIP_ALGO_WINOGRAD_LARGE) ||
      direction == SNN_HIP_FILTER_BACKPROP || p.input_format != 0 ||
      !conv2d_winograd_fused_supports(direction, p))
    return SNN_HIP_OK;
  size_t required = 0, recommended = 0;
  workspace_size(p, direction, algorithm, SNN_HIP_DTYPE_F32, &required,
                 &recommended);
  if (workspace == nullptr || workspace_elems < required)
    return SNN_HIP_INSUFFICIENT_WORKSPACE;
  LaunchOptions options;
  options.prepare_only = true;
  return launch_conv2d_winograd_fused_f32(direction, nullptr, filter, nullptr,
                                          p, workspace, workspace_elems,
                                          as_stream(stream), &options);
}

int snn_hip_conv2d_prepared_f32(int direction, const float* input,
                                const float* filter, float* output,
                                const snn_hip_conv2d_params* params,
                                int algorithm, float* workspace,
                                size_t workspace_elems, void* stream) {
  if (direction < SNN_HIP_FORWARD || direction > SNN_HIP_FILTER_BACKPROP)
    return SNN_HIP_INVALID_PARAMETER;
  LaunchOptions options;
  options.filter_prepared = true;
  return conv2d_dispatch<float>(direction, input, filter, output, params,
                                algorithm, workspace, workspace_elems, stream,
                                &options);
}

int snn_hip_conv2d_workspace_size(const snn_hip_conv2d_params* params,
                                  int direction, int algorithm,
                                  size_t* required_elems,
                                  size_t* recommended_elems) {
  if (params == nullptr || required_elems == nullptr ||
      recommended_elems == nullptr)
    return SNN_HIP_INVALID_PARAMETER;
  if (direction < SNN_HIP_FORWARD || direction > SNN_HIP_FILTER_BACKPROP)
    return SNN_HIP_INVALID_PARAMETER;
  return workspace_size(*params, direction, algorithm, SNN_HIP_DTYPE_F32,
                        required_elems, recommended_elems);
}

int snn_hip_conv2d_workspace_size_for(const snn_hip_conv2d_params* params,
                                      int direction, int algorithm, int dtype,
                                      size_t* required_elems,
                                      size_t* recommended_elems) {
  if (params == nullptr || required_elems == nullptr ||
      recommended_elems == nullptr)
    return SNN_HIP_INVALID_PARAMETER;
  if (direction < SNN_HIP_FORWARD || direction > SNN_HIP_FILTER_BACKPROP)
    return SNN_HIP_INVALID_PARAMETER;
  if (dtype != SNN_HIP_DTYPE_F32 && dtype != SNN_HIP_DTYPE_F16)
    return SNN_HIP_INVALID_PARAMETER;
  return workspace_size(*params, direction, algorithm, dtype, required_elems,
                        recommended_elems);
}

int snn_hip_conv2d_algorithm_supports(const snn_hip_conv2d_params* params,
                                      int direction, int algorithm) {
  if (params == nullptr) return SNN_HIP_ALGO_NOT_SUPPORTED;
  return algorithm_supports(*params, direction, algorithm);
}

int snn_hip_conv2d_default_algorithm(const snn_hip_conv2d_params* params,
                                     int direction) {
  if (params == nullptr) return SNN_HIP_ALGO_NOT_SUPPORTED;
  return default_algorithm(*params, direction, SNN_HIP_DTYPE_F32);
}

int snn_hip_conv2d_default_algorithm_for(const snn_hip_conv2d_params* params,
                                         int direction, int dtype) {
  if (params == nullptr ||
      (dtype != SNN_HIP_DTYPE_F32 && dtype != SNN_HIP_DTYPE_F16))
    return SNN_HIP_ALGO_NOT_SUPPORTED;
  return default_algorithm(*params, direction, dtype);
}

int snn_hip_depthwise_conv2d_forward_f32(
    const float* input, const float* filter, float* output,
    const snn_hip_depthwise_params* params, void* stream) {
  return depthwise_dispatch<float>(SNN_HIP_FORWARD, input, filter, output,
                                   params, stream);
}

int snn_hip_depthwise_conv2d_input_backprop_f32(
    const float* input, const float* filter, float* output,
    const snn_hip_depthwise_params* params, void* stream) {
  return depthwise_dispatch<float>(SNN_HIP_INPUT_BACKPROP, input, filter,
                                   output, params, stream);
}

int snn_hip_depthwise_conv2d_filter_backprop_f32(
    const float* input, const float* filter, float* output,
    const snn_hip_depthwise_params* params, void* stream) {
  return depthwise_dispatch<float>(SNN_HIP_FILTER_BACKPROP, input, filter,
                                   output, params, stream);
}

int snn_hip_depthwise_conv2d_filter_backprop_noalloc_f32(
    const float* input, const float* filter, float* output,
    const snn_hip_depthwise_params* params, void* stream) {
  if (params == nullptr) return SNN_HIP_INVALID_PARAMETER;
  const int v = validate(*params);
  if (v != SNN_HIP_OK) return v;
  if (input == nullptr || filter == nullptr || output == nullptr)
    return SNN_HIP_INVALID_PARAMETER;
  const snn_hip_depthwise_params& p = *params;
  const size_t cm = static_cast<size_t>(p.channels) * p.channel_multiplier;
  if (!fits_int32(static_cast<size_t>(p.batch) * p.in_rows * p.in_cols *
                  p.channels) ||
      !fits_int32(static_cast<size_t>(p.batch) * p.out_rows * p.out_cols * cm))
    return SNN_HIP_INDEX_EXCEEDED;
  return launch_depthwise_filter_backprop_noalloc_f32(input, filter, output, p,
                                                      as_stream(stream));
}

int snn_hip_depthwise_conv2d_forward_f16(
    const void* input, const void* filter, void* output,
    const snn_hip_depthwise_params* params, void* stream) {
  return depthwise_dispatch<_Float16>(
      SNN_HIP_FORWARD, static_cast<const _Float16*>(input),
      static_cast<const _Float16*>(filter), static_cast<_Float16*>(output),
      params, stream);
}

int snn_hip_depthwise_conv2d_input_backprop_f16(
    const void* input, const void* filter, void* output,
    const snn_hip_depthwise_params* params, void* stream) {
  return depthwise_dispatch<_Float16>(
      SNN_HIP_INPUT_BACKPROP, static_cast<const _Float16*>(input),
      static_cast<const _Float16*>(filter), static_cast<_Float16*>(output),
      params, stream);
}

int snn_hip_depthwise_conv2d_filter_backprop_f16(
    const void* input, const void* filter, void* output,
    const snn_hip_depthwise_params* params, void* stream) {
  return depthwise_dispatch<_Float16>(
      SNN_HIP_FILTER_BACKPROP, static_cast<const _Float16*>(input),
      static_cast<const _Float16*>(filter), static_cast<_Float16*>(output),
      params, stream);
}

int snn_hip_pooling_forward_f32(const float* input, float* output,
                                const snn_hip_pooling_params* params, int op,
                                void* stream) {
  const int v = pooling_check(params, true);
  if (v != SNN_HIP_OK) return v;
  if (input == nullptr || output == nullptr) return SNN_HIP_INVALID_PARAMETER;
  return launch_pooling_forward<float>(input, output, *params, op,
                                       as_stream(stream));
}

int snn_hip_pooling_forward_f16(const void* input, void* output,
                                const snn_hip_pooling_params* params, int op,
                                void* stream) {
  const int v = pooling_check(params, true);
  if (v != SNN_HIP_OK) return v;
  if (input == nullptr || output == nullptr) return SNN_HIP_INVALID_PARAMETER;
  return launch_pooling_forward<_Float16>(
      static_cast<const _Float16*>(input), static_cast<_Float16*>(output),
      *params, op, as_stream(stream));
}

int snn_hip_pooling_max_grad_f32(const float* input_data,
                                 const float* output_data,
                                 const float* input_backprop,
                                 float* output_backprop,
                                 const snn_hip_pooling_params* params, int op,
                                 void* stream) {
  const int v = pooling_check(params, false);
  if (v != SNN_HIP_OK) return v;
  if (input_data == nullptr || output_data == nullptr ||
      input_backprop == nullptr || output_backprop == nullptr)
    return SNN_HIP_INVALID_PARAMETER;
  if (op != SNN_HIP_POOL_MAX && op != SNN_HIP_POOL_MAX_WITH_NAN)
    return SNN_HIP_INVALID_PARAMETER;
  return launch_pooling_max_grad(input_data, output_data, input_backprop,
                                 output_backprop, *params, op,
                                 as_stream(stream));
}

int snn_hip_pooling_avg_grad_f32(const float* input_backprop,
                                 float* output_backprop,
                                 const snn_hip_pooling_params* params,
                                 void* stream) {
  const int v = pooling_check(params, false);
  if (v != SNN_HIP_OK) return v;
  if (input_backprop == nullptr || output_backprop == nullptr)
    return SNN_HIP_INVALID_PARAMETER;
  return launch_pooling_avg_grad(input_backprop, output_backprop, *params,
                                 as_stream(stream));
}

int snn_hip_pooling_max_grad_f16(const void* input_data,
                                 const void* output_data,
                                 const void* input_backprop,
                                 void* output_backprop,
                                 const snn_hip_pooling_params* params, int op,
                                 void* stream) {
  const int v = pooling_check(params, false);
  if (v != SNN_HIP_OK) return v;
  if (input_data == nullptr || output_data == nullptr ||
      input_backprop == nullptr || output_backprop == nullptr)
    return SNN_HIP_INVALID_PARAMETER;
  if (op != SNN_HIP_POOL_MAX && op != SNN_HIP_POOL_MAX_WITH_NAN)
    return SNN_HIP_INVALID_PARAMETER;
  return launch_pooling_max_grad_f16(
      static_cast<const _Float16*>(input_data),
      static_cast<const _Float16*>(output_data),
      static_cast<const _Float16*>(input_backprop),
      static_cast<_Float16*>(output_backprop), *params, op,
      as_stream(stream));
}

int snn_hip_pooling_avg_grad_f16(const void* input_backprop,
                                 void* output_backprop,
                                 const snn_hip_pooling_params* params,
                                 void* stream) {
  const int v = pooling_check(params, false);
  if (v != SNN_HIP_OK) return v;
  if (input_backprop == nullptr || output_backprop == nullptr)
    return SNN_HIP_INVALID_PARAMETER;
  return launch_pooling_avg_grad_f16(
      static_cast<const _Float16*>(input_backprop),
      static_cast<_Float16*>(output_backprop), *params, as_stream(stream));
}

int snn_hip_matmul_f32(const float* lhs, const float* rhs, float* output,
                       int batches, int m, int k, int n, int transpose_lhs,
                       int transpose_rhs, float beta, void* stream) {
  if (lhs == nullptr || rhs == nullptr || output == nullptr)
    return SNN_HIP_INVALID_PARAMETER;
  // include/portdnn/matmul/launch.h validates positive sizes.
  if (batches <= 0 || m <= 0 || k <= 0 || n <= 0)
    return SNN_HIP_INVALID_PARAMETER;
  if (!fits_int32(static_cast<size_t>(batches) * m * k) ||
      !fits_int32(static_cast<size_t>(batches) * k * n) ||
      !fits_int32(static_cast<size_t>(batches) * m * n))
    return SNN_HIP_INDEX_EXCEEDED;
  return launch_matmul_f32(lhs, rhs, output, batches, m, k, n,
                           transpose_lhs != 0, transpose_rhs != 0, beta,
                           as_stream(stream));
}

int snn_hip_matmul_f16(const void* lhs, const void* rhs, void* output,
                       int batches, int m, int k, int n, int transpose_lhs,
                       int transpose_rhs, float beta, void* stream) {
  if (lhs == nullptr || rhs == nullptr || output == nullptr)
    return SNN_HIP_INVALID_PARAMETER;
  if (batches <= 0 || m <= 0 || k <= 0 || n <= 0)
    return SNN_HIP_INVALID_PARAMETER;
  if (!fits_int32(static_cast<size_t>(batches) * m * k) ||
      !fits_int32(static_cast<size_t>(batches) * k * n) ||
      !fits_int32(static_cast<size_t>(batches) * m * n))
    return SNN_HIP_INDEX_EXCEEDED;
  return launch_matmul_f16(static_cast<const _Float16*>(lhs),
                           static_cast<const _Float16*>(rhs),
                           static_cast<_Float16*>(output), batches, m, k, n,
                           transpose_lhs != 0, transpose_rhs != 0, beta,
                           as_stream(stream));
}

int snn_hip_conv2d_forward_bias_act_f32(
    const float* input, const float* filter, const float* bias, float* output,
    const snn_hip_conv2d_params* params, int algorithm, int activation,
    float* workspace, size_t workspace_elems, void* stream) {
  if (activation != SNN_HIP_ACTIVATION_NONE &&
      activation != SNN_HIP_ACTIVATION_RELU)
    return SNN_HIP_INVALID_PARAMETER;
  bool applied = false;
  LaunchOptions epilogue;
  epilogue.bias = bias;
  epilogue.relu = activation == SNN_HIP_ACTIVATION_RELU;
  epilogue.applied = &applied;
  const int status =
      conv2d_dispatch<float>(SNN_HIP_FORWARD, input, filter, output, params,
                             algorithm, workspace, workspace_elems, stream,
                             &epilogue);
  if (status != SNN_HIP_OK || applied || !epilogue.wanted()) return status;
  // The chosen kernel could not fold the epilogue into its stores (partial
  // sums meeting through atomics, the direct and three-stage kernels): one
  // in-place pass over the finished output.
  const size_t n = static_cast<size_t>(params->batch) * params->out_rows *
                   params->out_cols * params->features;
  return launch_bias_act_f32(output, bias, params->features, n, epilogue.relu,
                             as_stream(stream));
}

int snn_hip_scale_blend_f32(float* data, const float* prior, float alpha,
                            float beta, size_t n_items, void* stream) {
  if (data == nullptr || n_items == 0 || (beta != 0.f && prior == nullptr))
    return SNN_HIP_INVALID_PARAMETER;
  return launch_scale_blend_f32(data, prior, alpha, beta, n_items,
                                as_stream(stream));
}

int snn_hip_pointwise_forward_f32(const float* input, float* output,
                                  size_t n_items, int op, void* stream) {
  if (input == nullptr || output == nullptr || n_items == 0)
    return SNN_HIP_INVALID_PARAMETER;
  return launch_pointwise_forward_f32(op, input, output, n_items,
                                      as_stream(stream));
}

int snn_hip_pointwise_forward_f16(const void* input, void* output,
                                  size_t n_items, int op, void* stream) {
  if (input == nullptr || output == nullptr || n_items == 0)
    return SNN_HIP_INVALID_PARAMETER;
  return launch_pointwise_forward_f16(
      op, static_cast<const _Float16*>(input), static_cast<_Float16*>(output),
      n_items, as_stream(stream));
}

int snn_hip_pointwise_grad_f32(const float* input_forward,
                               const float* input_backprop,
                               float* output_backprop, size_t n_items, int op,
                               void* stream) {
  if (input_forward == nullptr || input_backprop == nullptr ||
      output_backprop == nullptr || n_items == 0)
    return SNN_HIP_INVALID_PARAMETER;
  return launch_pointwise_grad_f32(op, input_forward, input_backprop,
                                   output_backprop, n_items, as_stream(stream));
}

int snn_hip_pointwise_grad_f16(const void* input_forward,
                               const void* input_backprop,
                               void* output_backprop, size_t n_items, int op,
                               void* stream) {
  if (input_forward == nullptr || input_backprop == nullptr ||
      output_backprop == nullptr || n_items == 0)
    return SNN_HIP_INVALID_PARAMETER;
  return launch_pointwise_grad_f16(
      op, static_cast<const _Float16*>(input_forward),
      static_cast<const _Float16*>(input_backprop),
      static_cast<_Float16*>(output_backprop), n_items, as_stream(stream));
}

int snn_hip_binaryop_f32(const float* lhs, const float* rhs, float* output,
                         const int* lhs_dims, int n_lhs_dims,
                         const int* rhs_dims, int n_rhs_dims, int op,
                         void* stream) {
  if (lhs == nullptr || rhs == nullptr || output == nullptr ||
      (n_lhs_dims > 0 && lhs_dims == nullptr) ||
      (n_rhs_dims > 0 && rhs_dims == nullptr))
    return SNN_HIP_INVALID_PARAMETER;
  return launch_binaryop_f32(op, lhs, rhs, output, lhs_dims, n_lhs_dims,
                             rhs_dims, n_rhs_dims, as_stream(stream));
}

int snn_hip_binaryop_f16(const void* lhs, const void* rhs, void* output,
                         const int* lhs_dims, int n_lhs_dims,
                         const int* rhs_dims, int n_rhs_dims, int op,
                         void* stream) {
  if (lhs == nullptr || rhs == nullptr || output == nullptr ||
      (n_lhs_dims > 0 && lhs_dims == nullptr) ||
      (n_rhs_dims > 0 && rhs_dims == nullptr))
    return SNN_HIP_INVALID_PARAMETER;
  return launch_binaryop_f16(op, static_cast<const _Float16*>(lhs),
                             static_cast<const _Float16*>(rhs),
                             static_cast<_Float16*>(output), lhs_dims,
                             n_lhs_dims, rhs_dims, n_rhs_dims,
                             as_stream(stream));
}

}  // extern "C"
