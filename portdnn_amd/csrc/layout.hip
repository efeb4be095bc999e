// Layout conversions for callers that hold NCHW activations and FCHW filters
// (the layouts of cuDNN-style code, include/portdnn/data_format.h:33-46 and
// include/portdnn/filter_format.h:32-54).  portDNN computes such a
// convolution with dedicated NCHW direct kernels
// (src/conv2d/direct/kernels_nchw.h); here the operands are rewritten to
// NHWC / HWCF, which every kernel of this library is built for, and the
// result is written back in the caller's layout.
#include "snn_kernels.h"

namespace snn {
namespace {

constexpr int kTile = 32;

// out[b][c][r] = in[b][r][c]: a 32 x 32 tile goes through LDS so that both
// the reads and the writes are contiguous.
__global__ void __launch_bounds__(kTile * 8)
    transpose_batched_kernel(const float* __restrict__ in,
                             float* __restrict__ out, int rows, int cols) {
  __shared__ float tile[kTile][kTile + 1];
  const size_t base = static_cast<size_t>(blockIdx.z) * rows * cols;
  const int c0 = blockIdx.x * kTile, r0 = blockIdx.y * kTile;
  const int tx = threadIdx.x & (kTile - 1), ty = threadIdx.x / kTile;
#pragma unroll
  for (int i = ty; i < kTile; i += 8) {
    const int r = r0 + i, c = c0 + tx;
    if (r < rows && c < cols)
      tile[i][tx] = in[base + static_cast<size_t>(r) * cols + c];
  }
  __syncthreads();
#pragma unroll
  for (int i = ty; i < kTile; i += 8) {
    const int c = c0 + i, r = r0 + tx;
    if (r < rows && c < cols)
      out[base + static_cast<size_t>(c) * rows + r] = tile[tx][i];
  }
}

// FCHW [F][C][RS] <-> HWCF [RS][C][F]: filters are small, one element per
// lane with the destination index contiguous.
__global__ void __launch_bounds__(256)
    permute_filter_kernel(const float* __restrict__ in, float* __restrict__ out,
                          int features, int channels, int taps, int to_hwcf,
                          int n) {
  const int idx = blockIdx.x * 256 + threadIdx.x;
  if (idx >= n) return;
  if (to_hwcf) {
    const int f = idx % features;
    const int c = (idx / features) % channels;
    const int t = idx / (features * channels);
    out[idx] = in[(f * channels + c) * taps + t];
  } else {
    const int t = idx % taps;
    const int c = (idx / taps) % channels;
    const int f = idx / (taps * channels);
    out[idx] = in[(t * channels + c) * features + f];
  }
}

}  // namespace

int launch_transpose_batched_f32(const float* in, float* out, int batches,
                                 int rows, int cols, hipStream_t stream) {
  const dim3 grid(static_cast<unsigned>(ceil_div(cols, kTile)),
                  static_cast<unsigned>(ceil_div(rows, kTile)),
                  static_cast<unsigned>(batches));
  if (grid.y > 65535u || grid.z > 65535u) return SNN_HIP_INDEX_EXCEEDED;
  hipLaunchKernelGGL(transpose_batched_kernel, grid, dim3(kTile * 8), 0,
                     stream, in, out, rows, cols);
  const hipError_t e = hipGetLastError();
  return e == hipSuccess ? SNN_HIP_OK
                         : report_hip_error(e, "transpose_batched_kernel");
}

int launch_permute_filter_f32(const float* in, float* out, int features,
                              int channels, int taps, bool to_hwcf,
                              hipStream_t stream) {
  const int n = features * channels * taps;
  hipLaunchKernelGGL(permute_filter_kernel,
                     dim3(static_cast<unsigned>(ceil_div(n, 256))), dim3(256),
                     0, stream, in, out, features, channels, taps,
                     to_hwcf ? 1 : 0, n);
  const hipError_t e = hipGetLastError();
  return e == hipSuccess ? SNN_HIP_OK
                         : report_hip_error(e, "permute_filter_kernel");
}

}  // namespace snn
