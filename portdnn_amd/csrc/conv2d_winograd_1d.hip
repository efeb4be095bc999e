// One-dimensional Winograd F(2,3) for 1x3 and 3x1 stride-1 convolutions,
// forward and input backprop (gfx950, fp32): the counterpart of portDNN's
// <1,2,1,3> and <2,1,3,1> tilings
// (include/portdnn/internal/conv2d/winograd/launch.h:317-326 with the 1-D
// transforms of src/conv2d/winograd/kernels/tiles_impl.h).
//
// Along the window's axis two outputs come from four inputs with four
// multiplications instead of six:
//     v = Bt d = [d0 - d2, d1 + d2, d2 - d1, d1 - d3]
//     u = G g  = [g0, (g0 + g1 + g2) / 2, (g0 - g1 + g2) / 2, g2]
//     y = At (u .* v) = [m0 + m1 + m2, m1 - m2 - m3]
// (the same sign convention as the two-dimensional kernels).  A tile is one
// position of the other axis and two consecutive positions of the window's
// axis; the three stages are the filter transform, the input transform, four
// GEMMs M[xi] (tiles x K) = V[xi] (tiles x C) * U[xi] (C x K) on the MFMA
// kernel, and the output transform.  The workspace holds [U: 4 C K]
// [V: 4 T C][M: 4 T K], T the tiles of one minibatch of images.
//
// Input backprop is the forward algorithm on dY with the taps mirrored, the
// channel / feature roles swapped and padding 2 - pad along the axis.
#include "snn_kernels.h"

namespace snn {
namespace {

// The window's axis is described by element strides, so one set of kernels
// serves rows (3x1) and columns (1x3).
struct Geom1D {
  int batch;
  int in_len, out_len;      // along the window's axis
  int other;                // extent of the other axis (same in and out)
  int in_ch, out_ch;
  int pad;                  // before the first element, along the axis
  int tiles_len;            // ceil(out_len / 2)
  int n_tiles;              // batch * other * tiles_len
  // element strides (in channels units they are multiplied by the channel
  // count of the tensor in question)
  int in_axis_stride, in_other_stride;    // in pixels
  int out_axis_stride, out_other_stride;  // in pixels
};

// U[xi][cin][cout] = (G g)[xi]; g[t] = W[t][cin][cout], or for the input
// gradient g[t] = W[2 - t][cout][cin].
__global__ void __launch_bounds__(256)
    wino1d_filter_transform_kernel(const float* __restrict__ w,
                                   float* __restrict__ u, int channels,
                                   int features, bool backprop) {
  const int cin = backprop ? features : channels;
  const int cout = backprop ? channels : features;
  const int idx = blockIdx.x * 256 + threadIdx.x;
  if (idx >= cin * cout) return;
  const int co = idx % cout, ci = idx / cout;
  float g[3];
#pragma unroll
  for (int t = 0; t < 3; ++t)
    g[t] = backprop
               ? w[(static_cast<size_t>(2 - t) * channels + co) * features + ci]
               : w[(static_cast<size_t>(t) * channels + ci) * features + co];
  const size_t plane = static_cast<size_t>(cin) * cout;
  u[0 * plane + idx] = g[0];
  u[1 * plane + idx] = 0.5f * (g[0] + g[1] + g[2]);
  u[2 * plane + idx] = 0.5f * (g[0] - g[1] + g[2]);
  u[3 * plane + idx] = g[2];
}

__device__ inline void tile_position(const Geom1D& g, int tile, int* n,
                                     int* other, int* t) {
  *t = tile % g.tiles_len;
  const int rest = tile / g.tiles_len;
  *other = rest % g.other;
  *n = rest / g.other;
}

// V[xi][tile][c] = (Bt d)[xi]; one lane per (tile, channel), channel fastest.
__global__ void __launch_bounds__(256)
    wino1d_input_transform_kernel(const float* __restrict__ in,
                                  float* __restrict__ v, Geom1D g) {
  const size_t idx = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
  if (idx >= static_cast<size_t>(g.n_tiles) * g.in_ch) return;
  const int c = static_cast<int>(idx % g.in_ch);
  const int tile = static_cast<int>(idx / g.in_ch);
  int n, other, t;
  tile_position(g, tile, &n, &other, &t);
  const int a0 = 2 * t - g.pad;
  const size_t image = static_cast<size_t>(g.in_len) * g.other;
  const float* base =
      in + (static_cast<size_t>(n) * image +
            static_cast<size_t>(other) * g.in_other_stride) * g.in_ch + c;
  float d[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int a = a0 + i;
    d[i] = (a >= 0 && a < g.in_len)
               ? base[static_cast<size_t>(a) * g.in_axis_stride * g.in_ch]
               : 0.f;
  }
  const size_t plane = static_cast<size_t>(g.n_tiles) * g.in_ch;
  float* out = v + static_cast<size_t>(tile) * g.in_ch + c;
  out[0 * plane] = d[0] - d[2];
  out[1 * plane] = d[1] + d[2];
  out[2 * plane] = d[2] - d[1];
  out[3 * plane] = d[1] - d[3];
}

// The two outputs of a tile = At m, clipped to the image.
__global__ void __launch_bounds__(256)
    wino1d_output_transform_kernel(const float* __restrict__ m,
                                   float* __restrict__ out, Geom1D g) {
  const size_t idx = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
  if (idx >= static_cast<size_t>(g.n_tiles) * g.out_ch) return;
  const int k = static_cast<int>(idx % g.out_ch);
  const int tile = static_cast<int>(idx / g.out_ch);
  int n, other, t;
  tile_position(g, tile, &n, &other, &t);
  const size_t plane = static_cast<size_t>(g.n_tiles) * g.out_ch;
  const float* src = m + static_cast<size_t>(tile) * g.out_ch + k;
  const float m0 = src[0], m1 = src[plane], m2 = src[2 * plane],
              m3 = src[3 * plane];
  const size_t image = static_cast<size_t>(g.out_len) * g.other;
  float* dst = out +
               (static_cast<size_t>(n) * image +
                static_cast<size_t>(other) * g.out_other_stride +
                static_cast<size_t>(2 * t) * g.out_axis_stride) * g.out_ch + k;
  dst[0] = m0 + m1 + m2;
  if (2 * t + 1 < g.out_len)
    dst[static_cast<size_t>(g.out_axis_stride) * g.out_ch] = m1 - m2 - m3;
}

}  // namespace

bool conv2d_winograd_1d_supports(int direction,
                                 const snn_hip_conv2d_params& p) {
  if (direction == SNN_HIP_FILTER_BACKPROP) return false;
  if (p.stride_rows != 1 || p.stride_cols != 1) return false;
  const bool along_cols = p.window_rows == 1 && p.window_cols == 3;
  const bool along_rows = p.window_rows == 3 && p.window_cols == 1;
  if (!along_cols && !along_rows) return false;
  // the window is 1 wide on the other axis: no padding there
  if (along_cols)
    return p.pad_rows == 0 && p.pad_cols <= 2 && p.out_rows == p.in_rows;
  return p.pad_cols == 0 && p.pad_rows <= 2 && p.out_cols == p.in_cols;
}

size_t conv2d_winograd_1d_workspace(int direction,
                                    const snn_hip_conv2d_params& p,
                                    int images) {
  const bool along_cols = p.window_rows == 1;
  const bool backprop = direction == SNN_HIP_INPUT_BACKPROP;
  const int out_len = backprop ? (along_cols ? p.in_cols : p.in_rows)
                               : (along_cols ? p.out_cols : p.out_rows);
  const int other = along_cols ? p.in_rows : p.in_cols;
  const size_t tiles = static_cast<size_t>(other) * ceil_div(out_len, 2);
  return static_cast<size_t>(4) * p.channels * p.features +
         static_cast<size_t>(4) * images * tiles * (p.channels + p.features);
}

int launch_conv2d_winograd_1d_f32(int direction, const float* input,
                                  const float* filter, float* output,
                                  const snn_hip_conv2d_params& p,
                                  float* workspace, size_t workspace_elems,
                                  hipStream_t stream, bool deterministic) {
  const bool backprop = direction == SNN_HIP_INPUT_BACKPROP;
  const bool along_cols = p.window_rows == 1;
  Geom1D g;
  const int x_len = along_cols ? p.in_cols : p.in_rows;
  const int y_len = along_cols ? p.out_cols : p.out_rows;
  const int pad = along_cols ? p.pad_cols : p.pad_rows;
  g.in_len = backprop ? y_len : x_len;
  g.out_len = backprop ? x_len : y_len;
  g.other = along_cols ? p.in_rows : p.in_cols;
  g.in_ch = backprop ? p.features : p.channels;
  g.out_ch = backprop ? p.channels : p.features;
  g.pad = backprop ? 2 - pad : pad;
  g.tiles_len = ceil_div(g.out_len, 2);
  // NHWC: a step along columns is one pixel, along rows one row of pixels
  if (along_cols) {
    g.in_axis_stride = 1;  g.in_other_stride = g.in_len;
    g.out_axis_stride = 1; g.out_other_stride = g.out_len;
  } else {
    g.in_axis_stride = g.other;  g.in_other_stride = 1;
    g.out_axis_stride = g.other; g.out_other_stride = 1;
  }
  const size_t tiles_img = static_cast<size_t>(g.other) * g.tiles_len;
  const size_t u_elems = static_cast<size_t>(4) * g.in_ch * g.out_ch;
  const size_t per_image = 4 * tiles_img * (g.in_ch + g.out_ch);
  if (workspace == nullptr || workspace_elems < u_elems + per_image)
    return SNN_HIP_INSUFFICIENT_WORKSPACE;
  const int minibatch = static_cast<int>(
      min(static_cast<size_t>(p.batch), (workspace_elems - u_elems) / per_image));
  float* u = workspace;
  float* v = u + u_elems;
  float* m = v + static_cast<size_t>(4) * minibatch * tiles_img * g.in_ch;

  hipLaunchKernelGGL(wino1d_filter_transform_kernel,
                     dim3(ceil_div(g.in_ch * g.out_ch, 256)), dim3(256), 0,
                     stream, filter, u, p.channels, p.features, backprop);
  for (int first = 0; first < p.batch; first += minibatch) {
    g.batch = min(minibatch, p.batch - first);
    g.n_tiles = g.batch * static_cast<int>(tiles_img);
    const float* in_mb = input + static_cast<size_t>(first) * g.in_len *
                                     g.other * g.in_ch;
    float* out_mb = output + static_cast<size_t>(first) * g.out_len * g.other *
                                 g.out_ch;
    size_t n = static_cast<size_t>(g.n_tiles) * g.in_ch;
    hipLaunchKernelGGL(wino1d_input_transform_kernel,
                       dim3(static_cast<unsigned>(ceil_div(n, size_t{256}))),
                       dim3(256), 0, stream, in_mb, v, g);
    SNN_HIP_CHECK_LAUNCH();
    int rc;
    if (batched_gemm_mfma_supports(g.n_tiles, g.in_ch, g.out_ch, v, u, m))
      rc = launch_batched_gemm_mfma_f32(v, u, m, 4, g.n_tiles, g.in_ch,
                                        g.out_ch, stream, false, false,
                                        deterministic);
    else
      rc = launch_matmul_f32(v, u, m, 4, g.n_tiles, g.in_ch, g.out_ch, false,
                             false, 0.f, stream);
    if (rc != SNN_HIP_OK) return rc;
    n = static_cast<size_t>(g.n_tiles) * g.out_ch;
    hipLaunchKernelGGL(wino1d_output_transform_kernel,
                       dim3(static_cast<unsigned>(ceil_div(n, size_t{256}))),
                       dim3(256), 0, stream, m, out_mb, g);
    SNN_HIP_CHECK_LAUNCH();
  }
  return SNN_HIP_OK;
}

}  // namespace snn
