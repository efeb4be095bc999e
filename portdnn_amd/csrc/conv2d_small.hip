// Forward convolution of small problems (one or a few images) on MFMA: no
// atomics, no zero fill, one launch.  It stands in for the reference's small
// tile list of the tiled algorithm (src/conv2d/tiled/launch_tiled.cc:215-226),
// which exists for the same reason: a single 56x56x64 image has 3136 output
// pixels, 49 tiles of 64x64, far fewer than the GPU has compute units.
//
// Work decomposition.  A work-group of four waves owns 16 consecutive output
// pixels (images, rows and columns flattened) x 64 features, and the four
// waves split the *reduction*: wave w takes channels 16 w .. 16 w + 15 of every
// 64-channel group of every filter tap.  One single-image 56x56x64 layer is
// then 196 work-groups of 4 waves, each wave 144 matrix instructions, and the
// partial tiles of the four waves meet through 16 KiB of LDS -- in a fixed
// order, so the result is the same every run.
//
// Operands never touch LDS.  v_mfma_f32_16x16x4_f32 wants A[pixel l % 16][k =
// l / 16] and B[k = l / 16][column l % 16] in lane l.  In NHWC the 16 channels
// of a step are contiguous, so lane (m, q) loads channels 4 q .. 4 q + 3 of its
// pixel with one 16-byte load and uses component j in sub-step j, which makes
// sub-step j's reduction index k = 4 q + j.  In HWCF the features of one
// reduction row are contiguous, so lane (n, q) loads features 4 n .. 4 n + 3 of
// row (4 q + j) with one 16-byte load: its four components are the B operands
// of four matrix instructions whose columns interleave (instruction u owns
// features 4 n + u).  A step is therefore 1 + 4 vector loads and 16 matrix
// instructions, and a lane ends with four consecutive features of a pixel.
// Padding taps and rows past the last pixel are out-of-range buffer offsets,
// which read as zero.
#include "gemm_tile.h"
#include "snn_kernels.h"

namespace snn {
namespace {

typedef float float4v __attribute__((ext_vector_type(4)));
typedef unsigned int uint4v __attribute__((ext_vector_type(4)));

constexpr unsigned kOob = 0x7FFFFFF0u;
constexpr size_t kMaxBufferBytes = 0x7FFFFFF0u;
constexpr int kPixels = 16;    // output pixels per work-group
constexpr int kFeatures = 64;  // features per work-group
constexpr int kDepth = 9;      // steps whose loads are in flight ahead

struct SmallGeom {
  int in_rows, in_cols, channels;
  int out_rows, out_cols, features;
  int win_rows, win_cols;
  int stride_rows, stride_cols, pad_rows, pad_cols;
  int m_total;  // batch * out_rows * out_cols
  int groups;   // channels / 64
  int steps;    // win_rows * win_cols * groups
};

__device__ inline __amdgpu_buffer_rsrc_t rsrc_of(const void* p, unsigned bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, bytes,
                                           0x00020000);
}

__device__ inline float4v load4(__amdgpu_buffer_rsrc_t r, unsigned off) {
  return __builtin_bit_cast(float4v,
                            __builtin_amdgcn_raw_buffer_load_b128(r, off, 0, 0));
}

struct StepOperands {
  float4v a;
  float4v b[4];
};

template <bool EPILOGUE>
__global__ void __launch_bounds__(256)
    conv_small_kernel(const float* __restrict__ x, const float* __restrict__ w,
                      float* __restrict__ y, SmallGeom g, unsigned x_bytes,
                      unsigned w_bytes, unsigned y_bytes,
                      const float* __restrict__ bias, int relu) {
  __shared__ float part[4][16][64];
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int m = lane & 15, q = lane >> 4;
  const __amdgpu_buffer_rsrc_t x_rsrc = rsrc_of(x, x_bytes);
  const __amdgpu_buffer_rsrc_t w_rsrc = rsrc_of(w, w_bytes);
  const __amdgpu_buffer_rsrc_t y_rsrc = rsrc_of(y, y_bytes);
  const int f0 = blockIdx.y * kFeatures;

  // this lane's pixel for the A operand
  const int pix = blockIdx.x * kPixels + m;
  const bool pix_ok = pix < g.m_total;
  const int ox = pix % g.out_cols;
  const int rest = pix / g.out_cols;
  const int oy = rest % g.out_rows;
  const int n = rest / g.out_rows;
  const int iy0 = oy * g.stride_rows - g.pad_rows;
  const int ix0 = ox * g.stride_cols - g.pad_cols;
  // element offset of (n, iy0, ix0, this lane's first channel)
  const int c_lane = 16 * wave + 4 * q;
  const int x_base =
      ((n * g.in_rows + iy0) * g.in_cols + ix0) * g.channels + c_lane;
  // byte offset of W[tap 0][c_lane][f0 + 4 m]
  const unsigned w_base =
      static_cast<unsigned>(c_lane * g.features + f0 + 4 * m) * 4u;
  const unsigned w_row = static_cast<unsigned>(g.features) * 4u;

  auto fetch = [&](int step, StepOperands& o) {
    // step -> (tap row, tap column, channel group); wave-uniform arithmetic
    const int grp = step % g.groups;
    const int tap = step / g.groups;
    const int r = tap / g.win_cols, s = tap % g.win_cols;
    const bool ok = pix_ok && step < g.steps &&
                    static_cast<unsigned>(iy0 + r) <
                        static_cast<unsigned>(g.in_rows) &&
                    static_cast<unsigned>(ix0 + s) <
                        static_cast<unsigned>(g.in_cols);
    const unsigned xo =
        ok ? static_cast<unsigned>(x_base + (r * g.in_cols + s) * g.channels +
                                   64 * grp) * 4u
           : kOob;
    o.a = load4(x_rsrc, xo);
    const unsigned wo =
        step < g.steps
            ? w_base + static_cast<unsigned>(tap * g.channels + 64 * grp) * w_row
            : kOob;
#pragma unroll
    for (int j = 0; j < 4; ++j)
      o.b[j] = load4(w_rsrc, wo == kOob ? kOob : wo + j * w_row);
  };

  float4v acc[4];
#pragma unroll
  for (int u = 0; u < 4; ++u) acc[u] = float4v{0.f, 0.f, 0.f, 0.f};

  StepOperands ring[kDepth];
#pragma unroll
  for (int d = 0; d < kDepth; ++d) fetch(d, ring[d]);
  for (int s0 = 0; s0 < g.steps; s0 += kDepth) {
#pragma unroll
    for (int d = 0; d < kDepth; ++d) {
      // a step past the end multiplies zeros (its loads were out of range)
      const StepOperands cur = ring[d];
      fetch(s0 + d + kDepth, ring[d]);
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int u = 0; u < 4; ++u)
          acc[u] = __builtin_amdgcn_mfma_f32_16x16x4f32(cur.a[j], cur.b[j][u],
                                                        acc[u], 0, 0, 0);
    }
  }

  // acc[u][i] is (pixel 4 q + i, feature f0 + 4 m + u) of this wave's share of
  // the reduction.  Wave w sums row i = w of every 4-pixel group: one pixel,
  // four consecutive features per lane.
#pragma unroll
  for (int u = 0; u < 4; ++u)
#pragma unroll
    for (int i = 0; i < 4; ++i) part[wave][4 * i + u][lane] = acc[u][i];
  __syncthreads();
  float4v sum;
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    float v = part[0][4 * wave + u][lane];
#pragma unroll
    for (int ww = 1; ww < 4; ++ww) v += part[ww][4 * wave + u][lane];
    sum[u] = v;
  }
  if (EPILOGUE) {
    if (bias != nullptr) {
#pragma unroll
      for (int u = 0; u < 4; ++u) sum[u] += bias[f0 + 4 * m + u];
    }
    if (relu) {
#pragma unroll
      for (int u = 0; u < 4; ++u) sum[u] = fmaxf(sum[u], 0.f);
    }
  }
  const int out_pix = blockIdx.x * kPixels + 4 * q + wave;
  const unsigned yo =
      out_pix < g.m_total
          ? static_cast<unsigned>(out_pix * g.features + f0 + 4 * m) * 4u
          : kOob;
  __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(uint4v, sum),
                                         y_rsrc, yo, 0, 0);
}

}  // namespace

// Channel and feature counts in multiples of 64, tensors addressable with
// 32-bit byte offsets, and few enough output tiles that the large-tile
// kernels would leave most compute units idle (they split the reduction
// across work-groups and meet through float atomics instead).
bool conv2d_small_supports(const snn_hip_conv2d_params& p) {
  const size_t pixels = static_cast<size_t>(p.batch) * p.out_rows * p.out_cols;
  const size_t x_bytes = static_cast<size_t>(p.batch) * p.in_rows * p.in_cols *
                         p.channels * sizeof(float);
  const size_t w_bytes = static_cast<size_t>(p.window_rows) * p.window_cols *
                         p.channels * p.features * sizeof(float);
  const size_t y_bytes = pixels * p.features * sizeof(float);
  if (p.channels % 64 != 0 || p.features % 64 != 0) return false;
  if (x_bytes > kMaxBufferBytes || w_bytes > kMaxBufferBytes ||
      y_bytes > kMaxBufferBytes)
    return false;
  const size_t tiles64 =
      ceil_div(pixels, size_t{64}) * static_cast<size_t>(p.features / 64);
  // ... and enough work-groups of this kernel's own to cover half the GPU,
  // each with a reduction short enough (18 steps = 288 matrix instructions
  // per wave) that splitting it further would not pay
  const size_t groups =
      ceil_div(pixels, size_t{kPixels}) * static_cast<size_t>(p.features / 64);
  const int steps = p.window_rows * p.window_cols * (p.channels / 64);
  return tiles64 < 128 && groups >= 128 && steps <= 18;
}

// x, w, y 16-byte aligned.  `epilogue` (may be null): bias per feature and / or
// ReLU applied to the sums before they are stored.
int launch_conv2d_small_f32(const float* x, const float* w, float* y,
                            const snn_hip_conv2d_params& p, hipStream_t stream,
                            const LaunchOptions* epilogue) {
  if (!conv2d_small_supports(p)) return SNN_HIP_INVALID_ALGORITHM;
  SmallGeom g;
  g.in_rows = p.in_rows; g.in_cols = p.in_cols; g.channels = p.channels;
  g.out_rows = p.out_rows; g.out_cols = p.out_cols; g.features = p.features;
  g.win_rows = p.window_rows; g.win_cols = p.window_cols;
  g.stride_rows = p.stride_rows; g.stride_cols = p.stride_cols;
  g.pad_rows = p.pad_rows; g.pad_cols = p.pad_cols;
  g.m_total = p.batch * p.out_rows * p.out_cols;
  g.groups = p.channels / 64;
  g.steps = p.window_rows * p.window_cols * g.groups;
  const unsigned x_bytes = static_cast<unsigned>(
      static_cast<size_t>(p.batch) * p.in_rows * p.in_cols * p.channels * 4);
  const unsigned w_bytes = static_cast<unsigned>(
      static_cast<size_t>(p.window_rows) * p.window_cols * p.channels *
      p.features * 4);
  const unsigned y_bytes =
      static_cast<unsigned>(static_cast<size_t>(g.m_total) * p.features * 4);
  const dim3 grid(static_cast<unsigned>(ceil_div(g.m_total, kPixels)),
                  static_cast<unsigned>(p.features / kFeatures));
  const bool fold = epilogue != nullptr && epilogue->wanted();
  {
    KernelTimer timer(stream);
    if (fold)
      hipLaunchKernelGGL(conv_small_kernel<true>, grid, dim3(256), 0, stream, x,
                         w, y, g, x_bytes, w_bytes, y_bytes, epilogue->bias,
                         epilogue->relu ? 1 : 0);
    else
      hipLaunchKernelGGL(conv_small_kernel<false>, grid, dim3(256), 0, stream,
                         x, w, y, g, x_bytes, w_bytes, y_bytes, nullptr, 0);
  }
  SNN_HIP_CHECK_LAUNCH();
  if (fold && epilogue->applied != nullptr) *epilogue->applied = true;
  return SNN_HIP_OK;
}

}  // namespace snn
