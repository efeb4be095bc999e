// Filter gradient on the matrix cores (gfx950) with both operands loaded from
// memory straight into the matrix instruction's registers (fp32 tensors on the
// fp32 instruction; binary16 tensors on the binary16 instruction, see
// filter_backprop_direct_h16_kernel, or -- channel / feature counts that are
// not multiples of 4 -- converted on the way into the fp32 one; fp32 sums):
//   dW[r][s][c][k] = sum over output pixels m of X[m shifted by (r, s)][c] * dY[m][k]
// (portDNN: a matmul with the left operand transposed for 1x1 windows,
// src/conv2d/matmul, and the im2col / tiled filter-gradient kernels otherwise,
// include/portdnn/conv2d/launch.h:59-118 with conv_type::FilterBackprop).
//
// The reduction index (the pixel) is the slow dimension of both NHWC operands,
// which is exactly how v_mfma_f32_16x16x4_f32 wants them: lane l supplies
// A[row l % 16][k = l / 16] and B[k = l / 16][column l % 16], i.e. for both
// operands element [pixel m0 + l / 16][16 consecutive positions].  Letting row
// i of accumulator block e stand for channel c0 + 4 i + e (and column j of
// block f for feature k0 + 4 j + f) turns one 16-byte load per lane -- 4
// pixels x 64 consecutive channels per wave, 256 contiguous bytes per pixel --
// into the A operands of four blocks, and the same for dY.  So a wave owns a
// 64 x 64 tile of one filter tap of dW (4 x 4 blocks, 64 accumulators) and per
// step of 4 pixels issues two loads and 16 matrix instructions: no LDS, no
// barrier and no transposition anywhere in the reduction loop, and the
// operands stream from L2 into a rotation of register buffers a few steps
// ahead.  With a window the input pixel of a lane is the output pixel moved by
// the tap; taps that fall into the padding load zeros (offset out of range).
//
// The pixel range of a (tap, tile) unit is split over the 8 waves of a
// work-group, whose partial tiles meet in LDS and are added in wave order, and
// -- where there are fewer units than compute units -- over several
// work-groups, which write their sums as partial filters [split][R S C][K]
// (float atomics on dW measured 14 us per call for the million additions of a
// batch-32 layer) for a second kernel to add in a fixed order.  Either way the
// result is reproducible.
//
// Channel and feature counts that are not multiples of 64 leave the lanes of
// a tile that stick out loading zeros from out of range and their stores
// dropped; counts that are not multiples of 4 load and store element by
// element (VEC == 1) -- a slow way to feed the matrix cores, but the only
// alternative for such shapes is one lane per filter element.
#include <algorithm>
#include <cstdio>
#include <cstdlib>

#include "gemm_tile.h"
#include "snn_kernels.h"

namespace snn {
namespace {

using gemm::xcd_remap;

typedef float float4v __attribute__((ext_vector_type(4)));
typedef _Float16 half4v __attribute__((ext_vector_type(4)));
typedef unsigned int uint4v __attribute__((ext_vector_type(4)));
typedef unsigned int uint2v __attribute__((ext_vector_type(2)));
constexpr size_t kMaxBufferBytes = 0x7FFFFFF0u;
constexpr unsigned kOob = 0x7FFFFFF0u;
constexpr int kWaves = 8;         // shares of a work-group's pixel range
constexpr int kTile = 64;         // channels and features per tile
constexpr int kDepth = 4;         // steps of 4 pixels in flight per wave
                                  // (3 and 6 measured the same)
constexpr int kComputeUnits = 256;
constexpr int kMinStepsPerWave = 8;
constexpr size_t kLdsBytes = kWaves * kTile * kTile * sizeof(float);
constexpr double kMaxPartialBytes = 256.0 * 1024 * 1024;

struct XtDy {
  int m_total;         // output pixels: batch * out_rows * out_cols
  int channels, features;
  int c_tiles;         // ceil(channels / 64)
  int n_units;         // taps * c_tiles * ceil(features / 64)
  int steps_per_wave;  // steps of 4 pixels per wave
  // windows only
  int taps, win_cols;
  int in_rows, in_cols, out_rows, out_cols;
  int stride_rows, stride_cols, pad_rows, pad_cols;
};

__device__ inline __amdgpu_buffer_rsrc_t make_rsrc(const void* p,
                                                   unsigned bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, bytes,
                                           0x00020000);
}

// Four consecutive elements of T at byte offset `off` as floats.  VEC == 4:
// one load; VEC == 1: four, element e from out of range (zero) where dead[e]
// is all ones.
template <typename T, int VEC>
__device__ inline float4v load_four(__amdgpu_buffer_rsrc_t rsrc, unsigned off,
                                    const unsigned (&dead)[4]) {
  float4v r;
  if constexpr (VEC == 4) {
    if constexpr (sizeof(T) == 4) {
      r = __builtin_bit_cast(
          float4v, __builtin_amdgcn_raw_buffer_load_b128(rsrc, off, 0, 0));
    } else {
      const half4v h = __builtin_bit_cast(
          half4v, __builtin_amdgcn_raw_buffer_load_b64(rsrc, off, 0, 0));
#pragma unroll
      for (int e = 0; e < 4; ++e) r[e] = static_cast<float>(h[e]);
    }
  } else {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const unsigned o = (off + e * static_cast<unsigned>(sizeof(T))) | dead[e];
      if constexpr (sizeof(T) == 4) {
        r[e] = __builtin_bit_cast(
            float, __builtin_amdgcn_raw_buffer_load_b32(rsrc, o, 0, 0));
      } else {
        r[e] = static_cast<float>(__builtin_bit_cast(
            _Float16, __builtin_amdgcn_raw_buffer_load_b16(rsrc, o, 0, 0)));
      }
    }
  }
  return r;
}

// out = sum of the partial filters, in a fixed order, as T: COLS columns (of
// VEC floats) x 256 / COLS groups of splits per work-group (group g adds
// splits g, g + groups, ...), the groups meeting in LDS.
template <typename T, int VEC, int COLS>
__global__ void __launch_bounds__(256)
    filter_backprop_direct_reduce_kernel(const float* __restrict__ part,
                                         T* __restrict__ dw, unsigned n_cols,
                                         int splits) {
  constexpr int kGroups = 256 / COLS;
  __shared__ __align__(16) float sums[kGroups][COLS][VEC];
  const int col_l = threadIdx.x % COLS, sg = threadIdx.x / COLS;
  const unsigned col = blockIdx.x * COLS + col_l;
  const int mine = col < n_cols ? splits : 0;  // past the end: nothing to add
  float sum[VEC];
#pragma unroll
  for (int e = 0; e < VEC; ++e) sum[e] = 0.f;
#pragma unroll 4
  for (int s = sg; s < mine; s += kGroups) {
    const float* const src = part + (static_cast<size_t>(s) * n_cols + col) * VEC;
    if constexpr (VEC == 4) {
      const float4 v = *reinterpret_cast<const float4*>(src);
      sum[0] += v.x;
      sum[1] += v.y;
      sum[2] += v.z;
      sum[3] += v.w;
    } else {
      sum[0] += *src;
    }
  }
#pragma unroll
  for (int e = 0; e < VEC; ++e) sums[sg][col_l][e] = sum[e];
  __syncthreads();
  if (sg != 0 || col >= n_cols) return;
#pragma unroll
  for (int t = 1; t < kGroups; ++t)
#pragma unroll
    for (int e = 0; e < VEC; ++e) sum[e] += sums[t][col_l][e];
  T* const dst = dw + static_cast<size_t>(col) * VEC;
  if constexpr (VEC == 1) {
    *dst = static_cast<T>(sum[0]);
  } else if constexpr (sizeof(T) == 4) {
    *reinterpret_cast<float4*>(dst) = make_float4(sum[0], sum[1], sum[2], sum[3]);
  } else {
    half4v h;
#pragma unroll
    for (int e = 0; e < 4; ++e) h[e] = static_cast<_Float16>(sum[e]);
    *reinterpret_cast<half4v*>(dst) = h;
  }
}

// The 8 waves' partial tiles (acc[e][f][v]: channel c0 + 16 quad + 4 v + e,
// feature k0 + 4 l16 + f) meet in LDS and are added in wave order; the sum
// goes to `out` at this split's partial filter.
template <int VEC>
__device__ inline void reduce_and_store(const float4v (&acc)[4][4], float* lds,
                                        int wave, int tid, float* out,
                                        unsigned out_bytes, int split,
                                        unsigned split_bytes, int tap, int c0,
                                        int k0, const XtDy& g) {
  const int lane = tid & 63;
  const int l16 = lane & 15, quad = lane >> 4;
  // The 8 partial tiles meet in LDS: [wave][64 channels][64 features].
  float* const mine = lds + wave * (kTile * kTile);
#pragma unroll
  for (int e = 0; e < 4; ++e)
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      const int row = 16 * quad + 4 * v + e;
      *reinterpret_cast<float4*>(mine + row * kTile + 4 * l16) =
          make_float4(acc[e][0][v], acc[e][1][v], acc[e][2][v], acc[e][3][v]);
    }
  __syncthreads();
  const __amdgpu_buffer_rsrc_t out_rsrc = make_rsrc(out, out_bytes);
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int idx = tid + 64 * kWaves * i;  // float4 of the tile
    float4 sum = *reinterpret_cast<const float4*>(lds + 4 * idx);
#pragma unroll
    for (int w = 1; w < kWaves; ++w) {
      const float4 part =
          *reinterpret_cast<const float4*>(lds + w * (kTile * kTile) + 4 * idx);
      sum.x += part.x;
      sum.y += part.y;
      sum.z += part.z;
      sum.w += part.w;
    }
    const int row = idx >> 4, col = (idx & 15) * 4;
    const unsigned off =
        static_cast<unsigned>(split) * split_bytes +
        (static_cast<unsigned>(tap * g.channels + c0 + row) *
             static_cast<unsigned>(g.features) +
         static_cast<unsigned>(k0 + col)) * 4u;
    // (rows and columns past the end of a ragged tile: dropped, out of range)
    const bool row_live = c0 + row < g.channels;
    if constexpr (VEC == 4) {
      const bool live = row_live && k0 + col < g.features;
      __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(uint4v, sum),
                                             out_rsrc, live ? off : kOob, 0, 0);
    } else {
      const float vals[4] = {sum.x, sum.y, sum.z, sum.w};
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const bool live = row_live && k0 + col + e < g.features;
        __builtin_amdgcn_raw_buffer_store_b32(
            __builtin_bit_cast(unsigned, vals[e]), out_rsrc,
            live ? off + 4u * e : kOob, 0, 0);
      }
    }
  }
}

// `out` (fp32): dW, or the partial filters when a unit's pixels are split
// over work-groups or the tensors are binary16 (`split_bytes` apart, else 0).
// WINDOW: any window, stride and padding; otherwise 1x1, stride 1, unpadded,
// where X is one flat matrix.  VEC: 4 = channel and feature counts in
// multiples of 4 (vector loads and stores), 1 = any.
template <bool WINDOW, typename T, int VEC>
__global__ void __launch_bounds__(64 * kWaves)
    filter_backprop_direct_kernel(const T* __restrict__ x,
                                  const T* __restrict__ dy,
                                  float* __restrict__ out, XtDy g,
                                  unsigned x_bytes, unsigned out_bytes,
                                  unsigned split_bytes, unsigned n_groups) {
  extern __shared__ __align__(16) float lds[];
  constexpr unsigned kElem = sizeof(T);
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  // Units vary fastest (taps first): the work-groups an XCD runs side by side
  // share pixel ranges (and with them operand rows in its L2).
  const unsigned group = xcd_remap(blockIdx.x, n_groups);
  const int split = static_cast<int>(group / g.n_units);
  const int unit = static_cast<int>(group % g.n_units);
  const int tap = WINDOW ? unit % g.taps : 0;
  const int tile = WINDOW ? unit / g.taps : unit;
  const int c0 = (tile % g.c_tiles) * kTile;
  const int k0 = (tile / g.c_tiles) * kTile;

  const int share = split * kWaves + wave;
  const int m_begin = min(g.m_total, share * g.steps_per_wave * 4);
  const int m_end = min(g.m_total, m_begin + g.steps_per_wave * 4);
  const int n_steps = (m_end - m_begin + 3) >> 2;

  // Loads of dY past this wave's last pixel fall out of the buffer's range
  // and return zeros: the range ends where the wave's share ends (which also
  // cancels whatever X holds there).
  const unsigned x_row = static_cast<unsigned>(g.channels) * kElem;
  const unsigned y_row = static_cast<unsigned>(g.features) * kElem;
  const __amdgpu_buffer_rsrc_t x_rsrc =
      make_rsrc(x, WINDOW ? x_bytes : static_cast<unsigned>(m_end) * x_row);
  const __amdgpu_buffer_rsrc_t y_rsrc =
      make_rsrc(dy, static_cast<unsigned>(m_end) * y_row);
  const int l16 = lane & 15, quad = lane >> 4;
  const unsigned x_col = static_cast<unsigned>(c0 + 4 * l16) * kElem;
  // Channels / features past the end (counts that are not multiples of 64):
  // those lanes -- with VEC == 1 those elements -- load zeros from out of
  // range, and stay there.
  const bool x_live = c0 + 4 * l16 < g.channels;
  const bool y_live = k0 + 4 * l16 < g.features;
  unsigned x_dead_e[4], y_dead_e[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    x_dead_e[e] = c0 + 4 * l16 + e < g.channels ? 0u : ~0u;
    y_dead_e[e] = k0 + 4 * l16 + e < g.features ? 0u : ~0u;
  }
  unsigned vx = x_live
                    ? static_cast<unsigned>(m_begin + quad) * x_row + x_col
                    : kOob;
  unsigned vy = y_live ? static_cast<unsigned>(m_begin + quad) * y_row +
                             static_cast<unsigned>(k0 + 4 * l16) * kElem
                       : kOob;
  const unsigned x_step = x_live ? 4u * x_row : 0u;
  const unsigned y_step = y_live ? 4u * y_row : 0u;
  const unsigned x_dead = x_live ? 0u : ~0u;
  // windows: the output pixel this lane loads next, as (image, row, column),
  // and the tap's displacement
  int px_n = 0, px_y = 0, px_x = 0, tap_y = 0, tap_x = 0;
  if constexpr (WINDOW) {
    const int m = m_begin + quad;
    px_x = m % g.out_cols;
    const int t = m / g.out_cols;
    px_y = t % g.out_rows;
    px_n = t / g.out_rows;
    tap_y = tap / g.win_cols - g.pad_rows;
    tap_x = tap % g.win_cols - g.pad_cols;
  }

  float4v xa[kDepth], yb[kDepth];
  auto issue = [&](int d) {
    if constexpr (WINDOW) {
      const int iy = px_y * g.stride_rows + tap_y;
      const int ix = px_x * g.stride_cols + tap_x;
      // all ones where the tap falls outside the image (mask arithmetic: a
      // per-lane condition around the load would become a branch)
      const unsigned bad =
          x_dead |
          (0u - static_cast<unsigned>(
                    (static_cast<unsigned>(iy) >= static_cast<unsigned>(g.in_rows)) |
                    (static_cast<unsigned>(ix) >= static_cast<unsigned>(g.in_cols))));
      const unsigned off =
          static_cast<unsigned>((px_n * g.in_rows + iy) * g.in_cols + ix) * x_row +
          x_col;
      vx = (off & ~bad) | (kOob & bad);
      px_x += 4;
      while (px_x >= g.out_cols) {
        px_x -= g.out_cols;
        if (++px_y == g.out_rows) {
          px_y = 0;
          ++px_n;
        }
      }
    }
    xa[d] = load_four<T, VEC>(x_rsrc, vx, x_dead_e);
    yb[d] = load_four<T, VEC>(y_rsrc, vy, y_dead_e);
    if constexpr (!WINDOW) vx += x_step;
    vy += y_step;
  };
  float4v acc[4][4];
#pragma unroll
  for (int e = 0; e < 4; ++e)
#pragma unroll
    for (int f = 0; f < 4; ++f)
#pragma unroll
      for (int v = 0; v < 4; ++v) acc[e][f][v] = 0.f;
  auto multiply = [&](int d) {
#pragma unroll
    for (int e = 0; e < 4; ++e)
#pragma unroll
      for (int f = 0; f < 4; ++f)
        acc[e][f] = __builtin_amdgcn_mfma_f32_16x16x4f32(xa[d][e], yb[d][f],
                                                         acc[e][f], 0, 0, 0);
  };

  // (the scheduling barriers keep the loads in the order the loop's waits
  // count on: the oldest pair outstanding is the one multiplied next)
#pragma unroll
  for (int d = 0; d < kDepth; ++d) {
    issue(d);
    __builtin_amdgcn_sched_barrier(0);
  }
  int s = 0;
  for (; s + kDepth <= n_steps; s += kDepth) {
#pragma unroll
    for (int d = 0; d < kDepth; ++d) {
      __builtin_amdgcn_sched_barrier(0);
      multiply(d);
      __builtin_amdgcn_sched_barrier(0);
      issue(d);  // step s + d + kDepth (zeros past the end)
    }
  }
  __builtin_amdgcn_sched_barrier(0);
  const int rest = n_steps - s;
#pragma unroll
  for (int d = 0; d < kDepth - 1; ++d)
    if (d < rest) multiply(d);

  reduce_and_store<VEC>(acc, lds, wave, tid, out, out_bytes, split,
                        split_bytes, tap, c0, k0, g);
}

// Binary16 tensors with channel and feature counts in multiples of 4 on the
// binary16 matrix instruction: v_mfma_f32_16x16x16_f16 takes from lane l four
// consecutive reduction indices, A[row l % 16][4 (l / 16) .. + 3], so a step is
// 16 pixels and a lane loads, for each of ITS four pixels 4 (l / 16) + j, the
// 8 bytes of its four channels (features) and regroups the 4 x 4 halves in
// registers into one operand per accumulator block: eight loads, sixteen
// two-half packs and 16 matrix instructions per 16 pixels, against 64 matrix
// instructions of the fp32 form (whose products are the same: binary16 times
// binary16 is exact in fp32, and the sums are fp32 in both).  Tile, units,
// splits, partial filters and the reduction are those of the kernel above.
constexpr int kDepthH = 3;  // steps of 16 pixels in flight per wave

template <bool WINDOW>
__global__ void __launch_bounds__(64 * kWaves)
    filter_backprop_direct_h16_kernel(const _Float16* __restrict__ x,
                                      const _Float16* __restrict__ dy,
                                      float* __restrict__ out, XtDy g,
                                      unsigned x_bytes, unsigned out_bytes,
                                      unsigned split_bytes, unsigned n_groups) {
  extern __shared__ __align__(16) float lds[];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const unsigned group = xcd_remap(blockIdx.x, n_groups);
  const int split = static_cast<int>(group / g.n_units);
  const int unit = static_cast<int>(group % g.n_units);
  const int tap = WINDOW ? unit % g.taps : 0;
  const int tile = WINDOW ? unit / g.taps : unit;
  const int c0 = (tile % g.c_tiles) * kTile;
  const int k0 = (tile / g.c_tiles) * kTile;

  const int share = split * kWaves + wave;
  const int m_begin = min(g.m_total, share * g.steps_per_wave * 4);
  const int m_end = min(g.m_total, m_begin + g.steps_per_wave * 4);
  const int n_steps = (m_end - m_begin + 15) >> 4;

  // dY (and X without a window) past this wave's last pixel is out of the
  // buffer's range and loads zeros; with a window X's offsets are masked.
  const unsigned x_row = static_cast<unsigned>(g.channels) * 2u;
  const unsigned y_row = static_cast<unsigned>(g.features) * 2u;
  const __amdgpu_buffer_rsrc_t x_rsrc =
      make_rsrc(x, WINDOW ? x_bytes : static_cast<unsigned>(m_end) * x_row);
  const __amdgpu_buffer_rsrc_t y_rsrc =
      make_rsrc(dy, static_cast<unsigned>(m_end) * y_row);
  const int l16 = lane & 15, quad = lane >> 4;
  const unsigned x_col = static_cast<unsigned>(c0 + 4 * l16) * 2u;
  const bool x_live = c0 + 4 * l16 < g.channels;
  const bool y_live = k0 + 4 * l16 < g.features;
  int m_lane = m_begin + 4 * quad;  // the first of this lane's four pixels
  unsigned vx = x_live ? static_cast<unsigned>(m_lane) * x_row + x_col : kOob;
  unsigned vy = y_live ? static_cast<unsigned>(m_lane) * y_row +
                             static_cast<unsigned>(k0 + 4 * l16) * 2u
                       : kOob;
  const unsigned x_step = x_live ? 16u * x_row : 0u;
  const unsigned y_step = y_live ? 16u * y_row : 0u;
  const unsigned x_dead = x_live ? 0u : ~0u;
  int px_n = 0, px_y = 0, px_x = 0, tap_y = 0, tap_x = 0;
  if constexpr (WINDOW) {
    px_x = m_lane % g.out_cols;
    const int t = m_lane / g.out_cols;
    px_y = t % g.out_rows;
    px_n = t / g.out_rows;
    tap_y = tap / g.win_cols - g.pad_rows;
    tap_x = tap % g.win_cols - g.pad_cols;
  }

  uint2v hx[kDepthH][4], hy[kDepthH][4];
  auto issue = [&](int d) {
    unsigned ox[4];
    if constexpr (WINDOW) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int iy = px_y * g.stride_rows + tap_y;
        const int ix = px_x * g.stride_cols + tap_x;
        // all ones where the tap falls outside the image or the pixel is
        // past this wave's share (mask arithmetic, no branch around a load)
        const unsigned bad =
            x_dead |
            (0u - static_cast<unsigned>(
                      (static_cast<unsigned>(iy) >= static_cast<unsigned>(g.in_rows)) |
                      (static_cast<unsigned>(ix) >= static_cast<unsigned>(g.in_cols)) |
                      (m_lane + j >= m_end)));
        const unsigned off =
            static_cast<unsigned>((px_n * g.in_rows + iy) * g.in_cols + ix) *
                x_row + x_col;
        ox[j] = (off & ~bad) | (kOob & bad);
        // the next pixel
        const bool row_end = px_x + 1 == g.out_cols;
        const bool img_end = row_end & (px_y + 1 == g.out_rows);
        px_x = row_end ? 0 : px_x + 1;
        px_y = img_end ? 0 : px_y + (row_end ? 1 : 0);
        px_n += img_end ? 1 : 0;
      }
      // the other lanes' twelve pixels
      px_x += 12;
      while (px_x >= g.out_cols) {
        px_x -= g.out_cols;
        if (++px_y == g.out_rows) {
          px_y = 0;
          ++px_n;
        }
      }
      m_lane += 16;
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j) ox[j] = vx + static_cast<unsigned>(j) * x_row;
      vx += x_step;
    }
#pragma unroll
    for (int j = 0; j < 4; ++j)
      hx[d][j] = __builtin_bit_cast(
          uint2v, __builtin_amdgcn_raw_buffer_load_b64(x_rsrc, ox[j], 0, 0));
#pragma unroll
    for (int j = 0; j < 4; ++j)
      hy[d][j] = __builtin_bit_cast(
          uint2v, __builtin_amdgcn_raw_buffer_load_b64(
                      y_rsrc, vy + static_cast<unsigned>(j) * y_row, 0, 0));
    vy += y_step;
  };
  float4v acc[4][4];
#pragma unroll
  for (int e = 0; e < 4; ++e)
#pragma unroll
    for (int f = 0; f < 4; ++f)
#pragma unroll
      for (int v = 0; v < 4; ++v) acc[e][f][v] = 0.f;
  // element e of the four pixels' vectors, as one operand
  auto gather = [](const uint2v (&h)[4], int e) {
    half4v r;
#pragma unroll
    for (int j = 0; j < 4; ++j) r[j] = __builtin_bit_cast(half4v, h[j])[e];
    return r;
  };
  auto multiply = [&](int d) {
    half4v a[4], b[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      a[e] = gather(hx[d], e);
      b[e] = gather(hy[d], e);
    }
#pragma unroll
    for (int e = 0; e < 4; ++e)
#pragma unroll
      for (int f = 0; f < 4; ++f)
        acc[e][f] = __builtin_amdgcn_mfma_f32_16x16x16f16(a[e], b[f], acc[e][f],
                                                          0, 0, 0);
  };

#pragma unroll
  for (int d = 0; d < kDepthH; ++d) {
    issue(d);
    __builtin_amdgcn_sched_barrier(0);
  }
  int s = 0;
  for (; s + kDepthH <= n_steps; s += kDepthH) {
#pragma unroll
    for (int d = 0; d < kDepthH; ++d) {
      __builtin_amdgcn_sched_barrier(0);
      multiply(d);
      __builtin_amdgcn_sched_barrier(0);
      issue(d);  // step s + d + kDepthH (zeros past the end)
    }
  }
  __builtin_amdgcn_sched_barrier(0);
  const int rest = n_steps - s;
#pragma unroll
  for (int d = 0; d < kDepthH - 1; ++d)
    if (d < rest) multiply(d);

  reduce_and_store<4>(acc, lds, wave, tid, out, out_bytes, split, split_bytes,
                      tap, c0, k0, g);
}

struct Plan {
  XtDy g;
  int splits;   // work-groups per (tap, tile) unit
  bool window;  // anything but 1x1, stride 1, unpadded
  bool vec4;    // channels and features in multiples of 4
};

Plan make_plan(const snn_hip_conv2d_params& p) {
  Plan plan;
  XtDy& g = plan.g;
  g.m_total = p.batch * p.out_rows * p.out_cols;
  g.channels = p.channels;
  g.features = p.features;
  g.c_tiles = ceil_div(p.channels, kTile);
  g.taps = p.window_rows * p.window_cols;
  g.win_cols = p.window_cols;
  g.in_rows = p.in_rows;   g.in_cols = p.in_cols;
  g.out_rows = p.out_rows; g.out_cols = p.out_cols;
  g.stride_rows = p.stride_rows; g.stride_cols = p.stride_cols;
  g.pad_rows = p.pad_rows; g.pad_cols = p.pad_cols;
  g.n_units = g.taps * g.c_tiles * ceil_div(p.features, kTile);
  plan.window = g.taps != 1 || p.stride_rows != 1 || p.stride_cols != 1 ||
                p.pad_rows != 0 || p.pad_cols != 0 ||
                p.in_rows != p.out_rows || p.in_cols != p.out_cols;
  plan.vec4 = p.channels % 4 == 0 && p.features % 4 == 0;
  const int total_steps = ceil_div(g.m_total, 4);
  // Work-groups per unit: the count with the least estimated time.  A compute
  // unit holds one work-group (128 KB of LDS), so the launch runs in rounds of
  // 256; a wave's step is 16 matrix instructions of 32 cycles sharing a SIMD
  // with another wave (0.49 us), a round costs about 4 us of first loads and
  // LDS reduction on top, and partial filters are written and read back at
  // about 4 MB per us plus the second launch.  (The binary16 kernel's step
  // is about a third of that; a model with 0.17 us chose splits that measured
  // the same or up to 5 % slower on nine layers, so both share this one.)
  const double dw_bytes = 4.0 * g.taps * p.channels * p.features;
  const int max_splits = std::max(
      1, std::min({kComputeUnits, total_steps / (kWaves * kMinStepsPerWave),
                   static_cast<int>(kMaxPartialBytes / dw_bytes)}));
  int splits = 1;
  double best = -1;
  for (int sp = 1; sp <= max_splits; ++sp) {
    const int rounds = ceil_div(g.n_units * sp, kComputeUnits);
    const int steps = ceil_div(total_steps, sp * kWaves);
    double t = rounds * (steps * 0.49 + 4.0);
    if (sp > 1) t += 2.0 * sp * dw_bytes / 4e6 + 3.0;
    if (best < 0 || t < best) {
      best = t;
      splits = sp;
    }
  }
  g.steps_per_wave = ceil_div(total_steps, splits * kWaves);
  plan.splits = ceil_div(total_steps, g.steps_per_wave * kWaves);
  return plan;
}

bool supports(const snn_hip_conv2d_params& p, bool ragged, size_t elem) {
  // whole tiles, or (ragged) any counts
  if (!ragged && (p.channels % kTile != 0 || p.features % kTile != 0))
    return false;
  const size_t m = static_cast<size_t>(p.batch) * p.out_rows * p.out_cols;
  if (m < 4 * kWaves * kMinStepsPerWave) return false;
  // every byte offset a lane forms, prefetch past the end included
  const size_t rows = m + 16 * (kDepthH + 2);
  if (rows * p.features * elem > kMaxBufferBytes) return false;
  const size_t in_rows = static_cast<size_t>(p.batch + 1) * p.in_rows *
                             p.in_cols + 16 * (kDepthH + 2);
  if (in_rows * p.channels * elem > kMaxBufferBytes) return false;
  return static_cast<size_t>(p.window_rows) * p.window_cols * p.channels *
             p.features * sizeof(float) <= kMaxBufferBytes;
}

template <bool WINDOW, typename T, int VEC>
hipError_t launch_main(const T* x, const T* dy, float* out, const Plan& plan,
                       size_t x_bytes, unsigned out_bytes, unsigned split_bytes,
                       unsigned n_groups, hipStream_t stream) {
  static const hipError_t attr = hipFuncSetAttribute(
      reinterpret_cast<const void*>(filter_backprop_direct_kernel<WINDOW, T, VEC>),
      hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes);
  if (attr != hipSuccess) return attr;
  hipLaunchKernelGGL((filter_backprop_direct_kernel<WINDOW, T, VEC>),
                     dim3(n_groups), dim3(64 * kWaves), kLdsBytes, stream, x, dy,
                     out, plan.g, static_cast<unsigned>(x_bytes), out_bytes,
                     split_bytes, n_groups);
  return hipSuccess;
}

template <bool WINDOW>
hipError_t launch_main_h16(const _Float16* x, const _Float16* dy, float* out,
                           const Plan& plan, size_t x_bytes, unsigned out_bytes,
                           unsigned split_bytes, unsigned n_groups,
                           hipStream_t stream) {
  static const hipError_t attr = hipFuncSetAttribute(
      reinterpret_cast<const void*>(filter_backprop_direct_h16_kernel<WINDOW>),
      hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes);
  if (attr != hipSuccess) return attr;
  hipLaunchKernelGGL((filter_backprop_direct_h16_kernel<WINDOW>), dim3(n_groups),
                     dim3(64 * kWaves), kLdsBytes, stream, x, dy, out, plan.g,
                     static_cast<unsigned>(x_bytes), out_bytes, split_bytes,
                     n_groups);
  return hipSuccess;
}

template <typename T, int VEC>
void launch_reduce(const float* partial, T* dw, size_t dw_elems, int splits,
                   hipStream_t stream) {
  const unsigned n_cols = static_cast<unsigned>(dw_elems / VEC);
  // (few columns and many splits: narrower work-groups, more of them)
  if (n_cols / 64 >= 128 || splits <= 4)
    hipLaunchKernelGGL((filter_backprop_direct_reduce_kernel<T, VEC, 64>),
                       dim3(ceil_div(n_cols, 64u)), dim3(256), 0, stream,
                       partial, dw, n_cols, splits);
  else
    hipLaunchKernelGGL((filter_backprop_direct_reduce_kernel<T, VEC, 16>),
                       dim3(ceil_div(n_cols, 16u)), dim3(256), 0, stream,
                       partial, dw, n_cols, splits);
}

// T == float: dW written by the main kernel when one work-group owns a unit;
// otherwise partial filters and the reduce kernel (which also rounds to T).
template <typename T>
int launch(const T* x, const T* dy, T* dw, float* partial,
           const snn_hip_conv2d_params& p, hipStream_t stream) {
  const Plan plan = make_plan(p);
  const size_t dw_elems =
      static_cast<size_t>(plan.g.taps) * p.channels * p.features;
  const size_t x_bytes = static_cast<size_t>(p.batch) * p.in_rows * p.in_cols *
                         p.channels * sizeof(T);
  const unsigned n_groups = static_cast<unsigned>(plan.g.n_units) *
                            static_cast<unsigned>(plan.splits);
  const bool direct = sizeof(T) == 4 && plan.splits == 1;
  if (!direct && partial == nullptr) return SNN_HIP_INVALID_PARAMETER;
  float* const out = direct ? reinterpret_cast<float*>(dw) : partial;
  const unsigned out_bytes = static_cast<unsigned>(plan.splits * dw_elems * 4);
  const unsigned split_bytes =
      plan.splits > 1 ? static_cast<unsigned>(dw_elems * 4) : 0u;
  KernelTimer timer(stream);
  hipError_t err;
  if constexpr (sizeof(T) == 2) {
    if (plan.vec4 && SNN_TUNING_ENV("SNN_HIP_FBDIRECT_H16_OFF") == nullptr) {
      err = plan.window
                ? launch_main_h16<true>(x, dy, out, plan, x_bytes, out_bytes,
                                        split_bytes, n_groups, stream)
                : launch_main_h16<false>(x, dy, out, plan, x_bytes, out_bytes,
                                         split_bytes, n_groups, stream);
      if (err != hipSuccess) return SNN_HIP_DEVICE_ERROR;
      launch_reduce<T, 4>(partial, dw, dw_elems, plan.splits, stream);
      return SNN_HIP_OK;
    }
  }
  if (plan.window)
    err = plan.vec4 ? launch_main<true, T, 4>(x, dy, out, plan, x_bytes,
                                              out_bytes, split_bytes, n_groups,
                                              stream)
                    : launch_main<true, T, 1>(x, dy, out, plan, x_bytes,
                                              out_bytes, split_bytes, n_groups,
                                              stream);
  else
    err = plan.vec4 ? launch_main<false, T, 4>(x, dy, out, plan, x_bytes,
                                               out_bytes, split_bytes, n_groups,
                                               stream)
                    : launch_main<false, T, 1>(x, dy, out, plan, x_bytes,
                                               out_bytes, split_bytes, n_groups,
                                               stream);
  if (err != hipSuccess) return SNN_HIP_DEVICE_ERROR;
  if (!direct) {
    if (plan.vec4)
      launch_reduce<T, 4>(partial, dw, dw_elems, plan.splits, stream);
    else
      launch_reduce<T, 1>(partial, dw, dw_elems, plan.splits, stream);
  }
  return SNN_HIP_OK;
}

}  // namespace

bool conv2d_filter_backprop_direct_f32_supports(const snn_hip_conv2d_params& p,
                                                bool ragged) {
  return supports(p, ragged, sizeof(float));
}

bool conv2d_filter_backprop_direct_f16_supports(
    const snn_hip_conv2d_params& p) {
  return supports(p, true, sizeof(_Float16));
}

size_t conv2d_filter_backprop_direct_f32_partial_floats(
    const snn_hip_conv2d_params& p) {
  const Plan plan = make_plan(p);
  if (plan.splits == 1) return 0;
  return static_cast<size_t>(plan.splits) * plan.g.taps * p.channels *
         p.features;
}

size_t conv2d_filter_backprop_direct_f16_partial_floats(
    const snn_hip_conv2d_params& p) {
  const Plan plan = make_plan(p);
  return static_cast<size_t>(plan.splits) * plan.g.taps * p.channels *
         p.features;
}

int launch_conv2d_filter_backprop_direct_f32(const float* x, const float* dy,
                                             float* dw, float* partial,
                                             const snn_hip_conv2d_params& p,
                                             hipStream_t stream) {
  return launch<float>(x, dy, dw, partial, p, stream);
}

int launch_conv2d_filter_backprop_direct_f16(const _Float16* x,
                                             const _Float16* dy, _Float16* dw,
                                             float* partial,
                                             const snn_hip_conv2d_params& p,
                                             hipStream_t stream) {
  return launch<_Float16>(x, dy, dw, partial, p, stream);
}

}  // namespace snn
