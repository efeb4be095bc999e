// Winograd F(2x2,3x3) convolution for gfx950, forward and input backprop.
//
// Counterpart of portDNN's Winograd chain
// (include/portdnn/internal/conv2d/winograd/launch.h:63-264 with the tiles of
// src/conv2d/winograd/kernels/tiles_impl.h:70-240): transform the filter once,
// then per minibatch transform the input, run 16 independent GEMMs
// [tiles x C] * [C x K] on MFMA and transform the result back,
//
//     Y = At [ (G g Gt) .* (Bt d B) ] A
//     Bt = | 1  0 -1  0 |   G = | 1    0    0  |   At = | 1  1  1  0 |
//          | 0  1  1  0 |       | 1/2  1/2  1/2|        | 0  1 -1 -1 |
//          | 0 -1  1  0 |       | 1/2 -1/2  1/2|
//          | 0  1  0 -1 |       | 0    0    1  |
//
// The caller's workspace is laid out as the reference lays it out
// (winograd/launch.h:237-261): [U: 16*C*K][V: 16*T*C][M: 16*T*K] with T the
// tiles of one minibatch; a workspace smaller than the recommended size makes
// the launcher loop over minibatches of images.
//
// Input backprop is the forward algorithm applied to dY with the filter
// mirrored in both spatial axes and its channel / feature roles swapped, and
// padding window - 1 - pad (internal/conv2d/winograd/kernel_params.h:44-55).
#include "snn_kernels.h"

namespace snn {
namespace {

struct WinoGeom {
  int batch;                 // images in this launch (minibatch)
  int in_rows, in_cols, in_ch;
  int out_rows, out_cols, out_ch;
  int pad_rows, pad_cols;
  int tile_rows, tile_cols;  // ceil(out / 2)
  int n_tiles;               // batch * tile_rows * tile_cols
};

// U[xi][cin][cout] = (G g Gt)[xi] with g[r][s] = W[r][s][c][k], or, for the
// input gradient, g[r][s] = W[2-r][2-s][cout][cin].
__global__ void __launch_bounds__(256)
    wino_filter_transform_kernel(const float* __restrict__ w,
                                 float* __restrict__ u, int channels,
                                 int features, bool backprop) {
  const int idx = blockIdx.x * 256 + threadIdx.x;
  const int cin = backprop ? features : channels;
  const int cout = backprop ? channels : features;
  if (idx >= cin * cout) return;
  const int co = idx % cout, ci = idx / cout;
  float g[3][3];
#pragma unroll
  for (int r = 0; r < 3; ++r)
#pragma unroll
    for (int s = 0; s < 3; ++s) {
      g[r][s] = backprop
                    ? w[((static_cast<size_t>(2 - r) * 3 + (2 - s)) * channels +
                         co) * features + ci]
                    : w[((static_cast<size_t>(r) * 3 + s) * channels + ci) *
                            features + co];
    }
  float t[4][3];  // G g
#pragma unroll
  for (int s = 0; s < 3; ++s) {
    t[0][s] = g[0][s];
    t[1][s] = 0.5f * (g[0][s] + g[1][s] + g[2][s]);
    t[2][s] = 0.5f * (g[0][s] - g[1][s] + g[2][s]);
    t[3][s] = g[2][s];
  }
  const size_t plane = static_cast<size_t>(cin) * cout;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const float o0 = t[i][0];
    const float o1 = 0.5f * (t[i][0] + t[i][1] + t[i][2]);
    const float o2 = 0.5f * (t[i][0] - t[i][1] + t[i][2]);
    const float o3 = t[i][2];
    u[(i * 4 + 0) * plane + idx] = o0;
    u[(i * 4 + 1) * plane + idx] = o1;
    u[(i * 4 + 2) * plane + idx] = o2;
    u[(i * 4 + 3) * plane + idx] = o3;
  }
}

template <int VEC>
struct Vec;
template <>
struct Vec<1> {
  using type = float;
  __device__ static float zero() { return 0.f; }
};
template <>
struct Vec<4> {
  using type = float4;
  __device__ static float4 zero() { return make_float4(0.f, 0.f, 0.f, 0.f); }
};
__device__ inline float4 operator+(float4 a, float4 b) {
  return make_float4(a.x + b.x, a.y + b.y, a.z + b.z, a.w + b.w);
}
__device__ inline float4 operator-(float4 a, float4 b) {
  return make_float4(a.x - b.x, a.y - b.y, a.z - b.z, a.w - b.w);
}

// V[xi][tile][c] = (Bt d B)[xi]; one lane per (tile, channel vector), channel
// fastest so that both the patch reads and the 16 plane writes are coalesced.
template <int VEC>
__global__ void __launch_bounds__(256)
    wino_input_transform_kernel(const float* __restrict__ in,
                                float* __restrict__ v, WinoGeom g) {
  using V = typename Vec<VEC>::type;
  const int cv = g.in_ch / VEC;
  const size_t idx = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
  if (idx >= static_cast<size_t>(g.n_tiles) * cv) return;
  const int c = static_cast<int>(idx % cv) * VEC;
  const int tile = static_cast<int>(idx / cv);
  const int tx = tile % g.tile_cols;
  const int t2 = tile / g.tile_cols;
  const int ty = t2 % g.tile_rows;
  const int n = t2 / g.tile_rows;
  const int y0 = 2 * ty - g.pad_rows, x0 = 2 * tx - g.pad_cols;
  const float* base =
      in + static_cast<size_t>(n) * g.in_rows * g.in_cols * g.in_ch + c;
  V d[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int y = y0 + i, x = x0 + j;
      d[i][j] = (y >= 0 && y < g.in_rows && x >= 0 && x < g.in_cols)
                    ? *reinterpret_cast<const V*>(
                          base + (static_cast<size_t>(y) * g.in_cols + x) *
                                     g.in_ch)
                    : Vec<VEC>::zero();
    }
  V t[4][4];  // Bt d
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    t[0][j] = d[0][j] - d[2][j];
    t[1][j] = d[1][j] + d[2][j];
    t[2][j] = d[2][j] - d[1][j];
    t[3][j] = d[1][j] - d[3][j];
  }
  const size_t plane = static_cast<size_t>(g.n_tiles) * g.in_ch;
  float* out = v + static_cast<size_t>(tile) * g.in_ch + c;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    *reinterpret_cast<V*>(out + (i * 4 + 0) * plane) = t[i][0] - t[i][2];
    *reinterpret_cast<V*>(out + (i * 4 + 1) * plane) = t[i][1] + t[i][2];
    *reinterpret_cast<V*>(out + (i * 4 + 2) * plane) = t[i][2] - t[i][1];
    *reinterpret_cast<V*>(out + (i * 4 + 3) * plane) = t[i][1] - t[i][3];
  }
}

// Y tile = At m A, clipped to the image.
template <int VEC>
__global__ void __launch_bounds__(256)
    wino_output_transform_kernel(const float* __restrict__ m,
                                 float* __restrict__ out, WinoGeom g) {
  using V = typename Vec<VEC>::type;
  const int kv = g.out_ch / VEC;
  const size_t idx = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
  if (idx >= static_cast<size_t>(g.n_tiles) * kv) return;
  const int k = static_cast<int>(idx % kv) * VEC;
  const int tile = static_cast<int>(idx / kv);
  const int tx = tile % g.tile_cols;
  const int t2 = tile / g.tile_cols;
  const int ty = t2 % g.tile_rows;
  const int n = t2 / g.tile_rows;
  const size_t plane = static_cast<size_t>(g.n_tiles) * g.out_ch;
  const float* src = m + static_cast<size_t>(tile) * g.out_ch + k;
  V a[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
      a[i][j] = *reinterpret_cast<const V*>(src + (i * 4 + j) * plane);
  V t[2][4];  // At m
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    t[0][j] = a[0][j] + a[1][j] + a[2][j];
    t[1][j] = a[1][j] - a[2][j] - a[3][j];
  }
  const int oy = 2 * ty, ox = 2 * tx;
  float* dst = out +
               ((static_cast<size_t>(n) * g.out_rows + oy) * g.out_cols + ox) *
                   g.out_ch + k;
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    if (oy + i >= g.out_rows) break;
    const V y0 = t[i][0] + t[i][1] + t[i][2];
    const V y1 = t[i][1] - t[i][2] - t[i][3];
    float* row = dst + static_cast<size_t>(i) * g.out_cols * g.out_ch;
    *reinterpret_cast<V*>(row) = y0;
    if (ox + 1 < g.out_cols) *reinterpret_cast<V*>(row + g.out_ch) = y1;
  }
}

inline bool aligned16(const void* p) {
  return (reinterpret_cast<uintptr_t>(p) & 15u) == 0;
}

}  // namespace

bool conv2d_winograd_supports(int direction, const snn_hip_conv2d_params& p) {
  return direction != SNN_HIP_FILTER_BACKPROP && p.window_rows == 3 &&
         p.window_cols == 3 && p.stride_rows == 1 && p.stride_cols == 1 &&
         p.pad_rows <= 2 && p.pad_cols <= 2;
}

int launch_conv2d_winograd_f32(int direction, const float* input,
                               const float* filter, float* output,
                               const snn_hip_conv2d_params& p,
                               float* workspace, size_t workspace_elems,
                               hipStream_t stream, bool deterministic) {
  const bool backprop = direction == SNN_HIP_INPUT_BACKPROP;
  WinoGeom g;
  g.in_rows = backprop ? p.out_rows : p.in_rows;
  g.in_cols = backprop ? p.out_cols : p.in_cols;
  g.in_ch = backprop ? p.features : p.channels;
  g.out_rows = backprop ? p.in_rows : p.out_rows;
  g.out_cols = backprop ? p.in_cols : p.out_cols;
  g.out_ch = backprop ? p.channels : p.features;
  g.pad_rows = backprop ? 2 - p.pad_rows : p.pad_rows;
  g.pad_cols = backprop ? 2 - p.pad_cols : p.pad_cols;
  g.tile_rows = ceil_div(g.out_rows, 2);
  g.tile_cols = ceil_div(g.out_cols, 2);
  const size_t tiles_img = static_cast<size_t>(g.tile_rows) * g.tile_cols;
  const size_t u_elems = static_cast<size_t>(16) * g.in_ch * g.out_ch;
  const size_t per_image = 16 * tiles_img * (g.in_ch + g.out_ch);
  if (workspace_elems < u_elems + per_image)
    return SNN_HIP_INSUFFICIENT_WORKSPACE;
  const int minibatch = static_cast<int>(
      min(static_cast<size_t>(p.batch), (workspace_elems - u_elems) / per_image));
  float* u = workspace;
  float* v = u + u_elems;
  float* m = v + static_cast<size_t>(16) * minibatch * tiles_img * g.in_ch;

  hipLaunchKernelGGL(wino_filter_transform_kernel,
                     dim3(ceil_div(g.in_ch * g.out_ch, 256)), dim3(256), 0,
                     stream, filter, u, p.channels, p.features, backprop);
  const bool vec_ok = g.in_ch % 4 == 0 && g.out_ch % 4 == 0 &&
                      aligned16(input) && aligned16(output) &&
                      aligned16(workspace);
  for (int first = 0; first < p.batch; first += minibatch) {
    g.batch = min(minibatch, p.batch - first);
    g.n_tiles = g.batch * static_cast<int>(tiles_img);
    const float* in_mb = input + static_cast<size_t>(first) * g.in_rows *
                                     g.in_cols * g.in_ch;
    float* out_mb = output + static_cast<size_t>(first) * g.out_rows *
                                 g.out_cols * g.out_ch;
    if (vec_ok) {
      const size_t n = static_cast<size_t>(g.n_tiles) * (g.in_ch / 4);
      hipLaunchKernelGGL(wino_input_transform_kernel<4>,
                         dim3(static_cast<unsigned>(ceil_div(n, size_t{256}))),
                         dim3(256), 0, stream, in_mb, v, g);
    } else {
      const size_t n = static_cast<size_t>(g.n_tiles) * g.in_ch;
      hipLaunchKernelGGL(wino_input_transform_kernel<1>,
                         dim3(static_cast<unsigned>(ceil_div(n, size_t{256}))),
                         dim3(256), 0, stream, in_mb, v, g);
    }
    SNN_HIP_CHECK_LAUNCH();
    // 16 GEMMs  M[xi] (tiles x out_ch) = V[xi] (tiles x in_ch) * U[xi]
    int rc;
    if (vec_ok &&
        batched_gemm_mfma_supports(g.n_tiles, g.in_ch, g.out_ch, v, u, m)) {
      rc = launch_batched_gemm_mfma_f32(v, u, m, 16, g.n_tiles, g.in_ch,
                                        g.out_ch, stream, false, false,
                                        deterministic);
    } else {
      rc = launch_matmul_f32(v, u, m, 16, g.n_tiles, g.in_ch, g.out_ch, false,
                             false, 0.f, stream);
    }
    if (rc != SNN_HIP_OK) return rc;
    if (vec_ok) {
      const size_t n = static_cast<size_t>(g.n_tiles) * (g.out_ch / 4);
      hipLaunchKernelGGL(wino_output_transform_kernel<4>,
                         dim3(static_cast<unsigned>(ceil_div(n, size_t{256}))),
                         dim3(256), 0, stream, m, out_mb, g);
    } else {
      const size_t n = static_cast<size_t>(g.n_tiles) * g.out_ch;
      hipLaunchKernelGGL(wino_output_transform_kernel<1>,
                         dim3(static_cast<unsigned>(ceil_div(n, size_t{256}))),
                         dim3(256), 0, stream, m, out_mb, g);
    }
    SNN_HIP_CHECK_LAUNCH();
  }
  return SNN_HIP_OK;
}

}  // namespace snn
