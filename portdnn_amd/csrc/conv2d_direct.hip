// Algorithm::Direct: plain convolution kernels for any window and stride, all
// three directions.  They stand in for portDNN's DirectConv2D functors
// (src/conv2d/direct/kernels_nhwc.h:25-450) and are the general fallback; the
// MFMA paths take over for the shapes they cover.
//
// Mapping (64-wide wavefronts, NHWC):
//   forward         one lane per output element, feature index fastest: the 64
//                   lanes of a wave read 64 consecutive filter features
//                   (coalesced) and broadcast one input value.
//   input backprop  one lane per dX element, channel fastest; filter rows
//                   [r][s][c][0..K) are walked contiguously per lane.
//   filter backprop one work-group per (r, s, c) and 64-feature strip; four
//                   waves split the batch*out_rows*out_cols reduction and
//                   combine through LDS (deterministic, no atomics).
#include "snn_kernels.h"

namespace snn {
namespace {

template <typename T>
__global__ void __launch_bounds__(256)
    direct_forward_kernel(const T* __restrict__ in, const T* __restrict__ fil,
                          T* __restrict__ out, snn_hip_conv2d_params p,
                          size_t n_out) {
  const size_t idx = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (idx >= n_out) return;
  const int K = p.features, C = p.channels;
  const int k = static_cast<int>(idx % K);
  size_t pix = idx / K;
  const int ox = static_cast<int>(pix % p.out_cols);
  pix /= p.out_cols;
  const int oy = static_cast<int>(pix % p.out_rows);
  const int n = static_cast<int>(pix / p.out_rows);
  const T* in_n = in + static_cast<size_t>(n) * p.in_rows * p.in_cols * C;
  float acc = 0.f;
  for (int r = 0; r < p.window_rows; ++r) {
    const int y = oy * p.stride_rows - p.pad_rows + r;
    if (y < 0 || y >= p.in_rows) continue;
    for (int s = 0; s < p.window_cols; ++s) {
      const int x = ox * p.stride_cols - p.pad_cols + s;
      if (x < 0 || x >= p.in_cols) continue;
      const T* ip = in_n + (static_cast<size_t>(y) * p.in_cols + x) * C;
      const T* fp = fil + static_cast<size_t>(r * p.window_cols + s) * C * K + k;
      for (int c = 0; c < C; ++c) {
        acc = fmaf(Elem<T>::load(ip + c),
                   Elem<T>::load(fp + static_cast<size_t>(c) * K), acc);
      }
    }
  }
  out[idx] = Elem<T>::from_float(acc);
}

template <typename T>
__global__ void __launch_bounds__(256)
    direct_input_backprop_kernel(const T* __restrict__ dy,
                                 const T* __restrict__ fil, T* __restrict__ dx,
                                 snn_hip_conv2d_params p, size_t n_out) {
  const size_t idx = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (idx >= n_out) return;
  const int K = p.features, C = p.channels;
  const int c = static_cast<int>(idx % C);
  size_t pix = idx / C;
  const int x = static_cast<int>(pix % p.in_cols);
  pix /= p.in_cols;
  const int y = static_cast<int>(pix % p.in_rows);
  const int n = static_cast<int>(pix / p.in_rows);
  const T* dy_n = dy + static_cast<size_t>(n) * p.out_rows * p.out_cols * K;
  float acc = 0.f;
  for (int r = 0; r < p.window_rows; ++r) {
    const int ty = y + p.pad_rows - r;
    if (ty < 0 || ty % p.stride_rows) continue;
    const int oy = ty / p.stride_rows;
    if (oy >= p.out_rows) continue;
    for (int s = 0; s < p.window_cols; ++s) {
      const int tx = x + p.pad_cols - s;
      if (tx < 0 || tx % p.stride_cols) continue;
      const int ox = tx / p.stride_cols;
      if (ox >= p.out_cols) continue;
      const T* gp = dy_n + (static_cast<size_t>(oy) * p.out_cols + ox) * K;
      const T* fp =
          fil + (static_cast<size_t>(r * p.window_cols + s) * C + c) * K;
      for (int k = 0; k < K; ++k) {
        acc = fmaf(Elem<T>::load(gp + k), Elem<T>::load(fp + k), acc);
      }
    }
  }
  dx[idx] = Elem<T>::from_float(acc);
}

constexpr int kFilBkStrip = 64;   // features per work-group
constexpr int kFilBkSlices = 4;   // waves splitting the spatial reduction

template <typename T>
__global__ void __launch_bounds__(kFilBkStrip* kFilBkSlices)
    direct_filter_backprop_kernel(const T* __restrict__ in,
                                  const T* __restrict__ dy,
                                  T* __restrict__ dw, snn_hip_conv2d_params p) {
  __shared__ float partial[kFilBkSlices][kFilBkStrip];
  const int K = p.features, C = p.channels;
  const int lane = threadIdx.x % kFilBkStrip;
  const int slice = threadIdx.x / kFilBkStrip;
  const int k = blockIdx.y * kFilBkStrip + lane;
  int rsc = blockIdx.x;
  const int c = rsc % C;
  rsc /= C;
  const int s = rsc % p.window_cols;
  const int r = rsc / p.window_cols;
  const int n_pix = p.batch * p.out_rows * p.out_cols;
  float acc = 0.f;
  if (k < K) {
    for (int pix = slice; pix < n_pix; pix += kFilBkSlices) {
      const int ox = pix % p.out_cols;
      const int t = pix / p.out_cols;
      const int oy = t % p.out_rows;
      const int n = t / p.out_rows;
      const int y = oy * p.stride_rows - p.pad_rows + r;
      const int x = ox * p.stride_cols - p.pad_cols + s;
      if (y < 0 || y >= p.in_rows || x < 0 || x >= p.in_cols) continue;
      const float xv = Elem<T>::load(
          in + ((static_cast<size_t>(n) * p.in_rows + y) * p.in_cols + x) * C +
          c);
      const float gv = Elem<T>::load(dy + static_cast<size_t>(pix) * K + k);
      acc = fmaf(xv, gv, acc);
    }
  }
  partial[slice][lane] = acc;
  __syncthreads();
  if (slice == 0 && k < K) {
    float sum = partial[0][lane];
    for (int i = 1; i < kFilBkSlices; ++i) sum += partial[i][lane];
    dw[static_cast<size_t>(blockIdx.x) * K + k] = Elem<T>::from_float(sum);
  }
}

}  // namespace

template <typename T>
int launch_conv2d_direct(int direction, const T* input, const T* filter,
                         T* output, const snn_hip_conv2d_params& p,
                         hipStream_t stream) {
  constexpr int kBlock = 256;
  if (direction == SNN_HIP_FORWARD) {
    const size_t n_out =
        static_cast<size_t>(p.batch) * p.out_rows * p.out_cols * p.features;
    const unsigned grid = static_cast<unsigned>(ceil_div(n_out, size_t{kBlock}));
    hipLaunchKernelGGL(direct_forward_kernel<T>, dim3(grid), dim3(kBlock), 0,
                       stream, input, filter, output, p, n_out);
  } else if (direction == SNN_HIP_INPUT_BACKPROP) {
    const size_t n_out =
        static_cast<size_t>(p.batch) * p.in_rows * p.in_cols * p.channels;
    const unsigned grid = static_cast<unsigned>(ceil_div(n_out, size_t{kBlock}));
    hipLaunchKernelGGL(direct_input_backprop_kernel<T>, dim3(grid),
                       dim3(kBlock), 0, stream, input, filter, output, p,
                       n_out);
  } else {
    const dim3 grid(static_cast<unsigned>(p.window_rows * p.window_cols *
                                          p.channels),
                    static_cast<unsigned>(ceil_div(p.features, kFilBkStrip)));
    hipLaunchKernelGGL(direct_filter_backprop_kernel<T>, grid,
                       dim3(kFilBkStrip * kFilBkSlices), 0, stream, input,
                       filter, output, p);
  }
  SNN_HIP_CHECK_LAUNCH();
  return SNN_HIP_OK;
}

template int launch_conv2d_direct<float>(int, const float*, const float*,
                                         float*, const snn_hip_conv2d_params&,
                                         hipStream_t);
template int launch_conv2d_direct<_Float16>(int, const _Float16*,
                                            const _Float16*, _Float16*,
                                            const snn_hip_conv2d_params&,
                                            hipStream_t);

}  // namespace snn
