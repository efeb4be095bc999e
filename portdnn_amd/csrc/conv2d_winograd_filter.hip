// Winograd F(3x3,2x2) filter gradient in one pass over the data (gfx950,
// fp32): the MI355X counterpart of portDNN's FilterBackprop Winograd tiling
// (include/portdnn/internal/conv2d/winograd/launch.h:341-345 with the
// transforms of src/conv2d/winograd/kernels/tiles_impl.h:288-329,374-490).
//
//   dW = sum over 2x2 tiles of dY:  At [ (G g Gt) .* (Bt d B) ] A
//     d  4x4 patch of X at (2 ty - pad, 2 tx - pad), g the 2x2 tile of dY,
//     Bt = | 1  0 -1  0 |   G = | 1    0  |   At = | 1  1  1  0 |
//          | 0  1  1  0 |       | 1/2  1/2|        | 0  1 -1  0 |
//          | 0 -1  1  0 |       | 1/2 -1/2|        | 0  1  1  1 |
//          | 0 -1  0  1 |       | 0    1  |
//   (1-D check: m0 = (d0-d2) g0, m1 = (d1+d2)(g0+g1)/2, m2 = (d2-d1)(g0-g1)/2,
//    m3 = (d3-d1) g1 give y0 = d0 g0 + d1 g1, y1 = d1 g0 + d2 g1,
//    y2 = d2 g0 + d3 g1.)
//
// The 16 element-wise products per (tile, channel, feature) are 16 GEMMs
// M[xi] (C x K) += V[xi]^T (C x tiles) * U[xi] (tiles x K) whose reduction
// runs over the tiles; they execute 16/36 of the direct algorithm's
// multiplications on v_mfma_f32_32x32x2_f32.  Neither V nor U reaches memory:
//
//   * a work-group of 12 waves owns 32 channels x 64 features of dW and a
//     range of tiles, walked 16 tiles at a time;
//   * waves 8-11 gather each tile's 4x4 patch for a channel pair (zero-filling
//     buffer loads for the padding), apply Bt d B in registers and write
//     V[xi][channel][tile] to LDS -- tile innermost, so a multiplying lane
//     fetches four reduction steps of its channel with one ds_read_b128 --
//     and copy the raw 2x2 tiles of dY to LDS;
//   * waves 0-7 multiply: wave (w, h) owns the transformed row w (xi = 4w ..
//     4w+3) for feature half h, forms G g Gt for its row from the raw dY tile
//     in registers (six additions per four matrix instructions) and keeps
//     4 x (32 x 32) accumulators;
//   * V and the dY tiles are double buffered, one barrier per 16 tiles;
//   * at the end At m A is applied along xi's column index inside each lane
//     and along its row index across the waves through LDS.
//
// The tile range is split across work-groups so that about one work-group per
// CU runs; each writes its 9 x 32 x 64 partial filter to a slot of the
// caller's workspace and a second kernel adds the slots in a fixed order, so
// the result is the same from run to run.
#include "gemm_tile.h"
#include "snn_kernels.h"

namespace snn {
namespace {

using gemm::comp;
using gemm::float16v;

constexpr int kBC = 32;         // channels per work-group
constexpr int kBK = 64;         // features per work-group
constexpr int kStepTiles = 16;  // tiles per LDS stage
constexpr int kThreadsWf = 768;
constexpr unsigned kOob = 0x7FFFFFF0u;
constexpr size_t kMaxBufferBytes = 0x7FFFFFF0u;

constexpr int kVStage = 16 * kBC * kStepTiles;   // floats: 32 KiB
constexpr int kGStage = kStepTiles * 4 * kBK;    // floats: 16 KiB
constexpr int kStage = kVStage + kGStage;
constexpr size_t kLdsBytes = 2 * kStage * sizeof(float);  // 96 KiB

typedef unsigned int uint4v __attribute__((ext_vector_type(4)));

struct FilterGeom {
  int batch, in_rows, in_cols, channels;
  int out_rows, out_cols, features;
  int pad_rows, pad_cols;
  int tile_rows, tile_cols, n_tiles;
  int tiles_per_split;  // a multiple of kStepTiles
  int c_blocks, k_blocks;
};

__device__ inline __amdgpu_buffer_rsrc_t make_rsrc(const void* p,
                                                   unsigned bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, bytes,
                                           0x00020000);
}
__device__ inline float2 operator+(float2 a, float2 b) {
  return make_float2(a.x + b.x, a.y + b.y);
}
__device__ inline float2 operator-(float2 a, float2 b) {
  return make_float2(a.x - b.x, a.y - b.y);
}

__global__ void __launch_bounds__(kThreadsWf)
    wino_filter_backprop_kernel(const float* __restrict__ x,
                                const float* __restrict__ dy,
                                float* __restrict__ dst, FilterGeom g,
                                unsigned x_bytes, unsigned dy_bytes,
                                unsigned n_groups, size_t slot_elems) {
  extern __shared__ __align__(16) float lds[];  // 2 x [V stage | dY stage]

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

  // group = (split, channel block, feature block), blocks of one split
  // adjacent so that they meet in one XCD's L2 (they read the same tiles)
  const unsigned group = gemm::xcd_remap(blockIdx.x, n_groups);
  const int blocks = g.c_blocks * g.k_blocks;
  const int split = static_cast<int>(group) / blocks;
  const int blk = static_cast<int>(group) - split * blocks;
  const int cb = blk / g.k_blocks, kb = blk - cb * g.k_blocks;
  const int c0 = cb * kBC, k0 = kb * kBK;
  const int tile_begin = split * g.tiles_per_split;
  const int tile_end = min(g.n_tiles, tile_begin + g.tiles_per_split);
  const int n_steps = (tile_end - tile_begin + kStepTiles - 1) / kStepTiles;

  float16v acc[4];
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[j][v] = 0.f;

  if (wave >= 8) {
    // ---- gather + transform waves ----------------------------------------
    const __amdgpu_buffer_rsrc_t x_rsrc = make_rsrc(x, x_bytes);
    const __amdgpu_buffer_rsrc_t dy_rsrc = make_rsrc(dy, dy_bytes);
    const int gt = tid - 512;
    const int tile_l = gt >> 4;  // 0 .. 15
    const int sub = gt & 15;     // channel pair of the patch / feature quad of dY
    // position of this lane's tile, advanced by kStepTiles per step
    int tile = tile_begin + tile_l;
    int tx = tile % g.tile_cols;
    int t2 = tile / g.tile_cols;
    int ty = t2 % g.tile_rows;
    int n = t2 / g.tile_rows;
    const unsigned x_ch_off = static_cast<unsigned>(c0 + 2 * sub) * 4u;
    const bool c_ok = c0 + 2 * sub < g.channels;
    const unsigned dy_f_off = static_cast<unsigned>(k0 + 4 * sub) * 4u;
    const bool f_ok = k0 + 4 * sub < g.features;

    struct Loaded {
      float2 d[16];
      float4 q[4];
    };
    auto load_step = [&](Loaded& r) {
      const bool live = tile < tile_end;
      const int y0 = 2 * ty - g.pad_rows, x0 = 2 * tx - g.pad_cols;
      const int img = n * g.in_rows;
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int yy = y0 + i, xx = x0 + j;
          const bool ok = live & c_ok &
                          (static_cast<unsigned>(yy) <
                           static_cast<unsigned>(g.in_rows)) &
                          (static_cast<unsigned>(xx) <
                           static_cast<unsigned>(g.in_cols));
          const unsigned off =
              ok ? static_cast<unsigned>(((img + yy) * g.in_cols + xx) *
                                         g.channels) * 4u + x_ch_off
                 : kOob;
          r.d[i * 4 + j] = __builtin_bit_cast(
              float2, __builtin_amdgcn_raw_buffer_load_b64(x_rsrc, off, 0, 0));
        }
      const int oimg = n * g.out_rows;
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          const int oy = 2 * ty + i, ox = 2 * tx + j;
          const bool ok = live & f_ok & (oy < g.out_rows) & (ox < g.out_cols);
          const unsigned off =
              ok ? static_cast<unsigned>(((oimg + oy) * g.out_cols + ox) *
                                         g.features) * 4u + dy_f_off
                 : kOob;
          r.q[i * 2 + j] = __builtin_bit_cast(
              float4, __builtin_amdgcn_raw_buffer_load_b128(dy_rsrc, off, 0, 0));
        }
      // next step's tile
      tile += kStepTiles;
      tx += kStepTiles;
      while (tx >= g.tile_cols) {
        tx -= g.tile_cols;
        if (++ty == g.tile_rows) {
          ty = 0;
          ++n;
        }
      }
    };
    // V[xi][channel][tile]: 16 tiles per row, the 16-byte group index xor-ed
    // with (channel / 2) % 4 so that the 16 lanes of a ds_read_b128 pass
    // (consecutive channels, one group) spread over all banks.
    float* const v_store = lds + (2 * sub) * kStepTiles +
                           4 * ((tile_l >> 2) ^ (sub & 3)) + (tile_l & 3);
    float* const g_store = lds + kVStage + tile_l * (4 * kBK) + 4 * sub;
    auto transform_store = [&](const Loaded& r, int buf) {
      float* const dst_v = v_store + buf * kStage;
      float2 t[4][4];  // Bt d
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        t[0][j] = r.d[0 * 4 + j] - r.d[2 * 4 + j];
        t[1][j] = r.d[1 * 4 + j] + r.d[2 * 4 + j];
        t[2][j] = r.d[2 * 4 + j] - r.d[1 * 4 + j];
        t[3][j] = r.d[3 * 4 + j] - r.d[1 * 4 + j];
      }
      constexpr int kXi = kBC * kStepTiles;  // floats per xi plane
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float2 o0 = t[i][0] - t[i][2];
        const float2 o1 = t[i][1] + t[i][2];
        const float2 o2 = t[i][2] - t[i][1];
        const float2 o3 = t[i][3] - t[i][1];
        float* const p = dst_v + (i * 4) * kXi;
        p[0 * kXi] = o0.x; p[0 * kXi + kStepTiles] = o0.y;
        p[1 * kXi] = o1.x; p[1 * kXi + kStepTiles] = o1.y;
        p[2 * kXi] = o2.x; p[2 * kXi + kStepTiles] = o2.y;
        p[3 * kXi] = o3.x; p[3 * kXi + kStepTiles] = o3.y;
      }
      float* const dst_g = g_store + buf * kStage;
#pragma unroll
      for (int px = 0; px < 4; ++px)
        *reinterpret_cast<float4*>(dst_g + px * kBK) = r.q[px];
    };
    // Two register sets: loads run two steps ahead of the transform that
    // consumes them (steps past the end read nothing and are never stored).
    Loaded even, odd;
    load_step(even);
    load_step(odd);
    transform_store(even, 0);
    load_step(even);
    __syncthreads();
    for (int s = 0; s < n_steps; s += 2) {
      if (s + 1 < n_steps) transform_store(odd, 1);
      load_step(odd);
      __syncthreads();
      if (s + 1 >= n_steps) break;
      if (s + 2 < n_steps) transform_store(even, 0);
      load_step(even);
      __syncthreads();
    }
  } else {
    // ---- multiplying waves -------------------------------------------------
    const int w = wave & 3;   // transformed row: xi = 4w .. 4w+3
    const int h = wave >> 2;  // feature half
    const int c_l = lane & 31;
    const int half = lane >> 5;
    constexpr int kXi = kBC * kStepTiles;
    const float* const a_base =
        lds + (4 * w * kBC + c_l) * kStepTiles;
    const int swz = (c_l >> 1) & 3;
    const float* const g_base = lds + kVStage + h * 32 + c_l;
    __syncthreads();
    for (int s = 0; s < n_steps; ++s) {
      const float* const a_buf = a_base + (s & 1) * kStage;
      const float* const g_buf = g_base + (s & 1) * kStage;
#pragma unroll
      for (int pg = 0; pg < 2; ++pg) {
        const int grp = 2 * pg + half;  // tiles 4 grp .. 4 grp + 3
        float4 a[4];
#pragma unroll
        for (int j = 0; j < 4; ++j)
          a[j] = *reinterpret_cast<const float4*>(a_buf + j * kXi +
                                                  4 * (grp ^ swz));
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          const float* const gp = g_buf + (4 * grp + t) * (4 * kBK);
          // row w of G g: g rows 0 and 1 are pixels (0,1) and (2,3)
          float h0, h1;
          if (w == 0) {
            h0 = gp[0 * kBK];
            h1 = gp[1 * kBK];
          } else if (w == 3) {
            h0 = gp[2 * kBK];
            h1 = gp[3 * kBK];
          } else {
            const float p00 = gp[0 * kBK], p01 = gp[1 * kBK];
            const float p10 = gp[2 * kBK], p11 = gp[3 * kBK];
            if (w == 1) {
              h0 = 0.5f * (p00 + p10);
              h1 = 0.5f * (p01 + p11);
            } else {
              h0 = 0.5f * (p00 - p10);
              h1 = 0.5f * (p01 - p11);
            }
          }
          const float u0 = h0, u1 = 0.5f * (h0 + h1), u2 = 0.5f * (h0 - h1),
                      u3 = h1;
          acc[0] = __builtin_amdgcn_mfma_f32_32x32x2f32(comp(a[0], t), u0,
                                                        acc[0], 0, 0, 0);
          acc[1] = __builtin_amdgcn_mfma_f32_32x32x2f32(comp(a[1], t), u1,
                                                        acc[1], 0, 0, 0);
          acc[2] = __builtin_amdgcn_mfma_f32_32x32x2f32(comp(a[2], t), u2,
                                                        acc[2], 0, 0, 0);
          acc[3] = __builtin_amdgcn_mfma_f32_32x32x2f32(comp(a[3], t), u3,
                                                        acc[3], 0, 0, 0);
        }
      }
      __syncthreads();
    }
    // At m A along xi's column index, inside the lane: three sums per row w.
    // exchange[w][h][s][v][lane]
    float* const e_base = lds + ((w * 2 + h) * 3 * 16) * 64 + lane;
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      e_base[(0 * 16 + v) * 64] = acc[0][v] + acc[1][v] + acc[2][v];
      e_base[(1 * 16 + v) * 64] = acc[1][v] - acc[2][v];
      e_base[(2 * 16 + v) * 64] = acc[1][v] + acc[2][v] + acc[3][v];
    }
  }
  __syncthreads();
  // Along xi's row index, across the waves; all 768 lanes write.  An item is
  // (h, s, v, lane): three outputs dW[r][s][channel][feature], r = 0 .. 2.
  float* const slot = dst + static_cast<size_t>(split) * slot_elems;
  const size_t plane = static_cast<size_t>(g.channels) * g.features;
  for (int item = tid; item < 2 * 3 * 16 * 64; item += kThreadsWf) {
    const int l = item & 63;
    const int v = (item >> 6) & 15;
    const int hs = item >> 10;  // h * 3 + s
    const int hh = hs / 3, s = hs - hh * 3;
    float m[4];
#pragma unroll
    for (int ww = 0; ww < 4; ++ww)
      m[ww] = lds[(((ww * 2 + hh) * 3 + s) * 16 + v) * 64 + l];
    const int c = c0 + 8 * (v >> 2) + 4 * (l >> 5) + (v & 3);
    const int f = k0 + hh * 32 + (l & 31);
    if (c < g.channels && f < g.features) {
      float* const o = slot + static_cast<size_t>(s) * plane +
                       static_cast<size_t>(c) * g.features + f;
      o[0 * 3 * plane] = m[0] + m[1] + m[2];
      o[1 * 3 * plane] = m[1] - m[2];
      o[2 * 3 * plane] = m[1] + m[2] + m[3];
    }
  }
}

// dW[e] = sum over the splits' partial filters.  A work-group adds up 16
// float4 elements: lane (slice, e) sums the splits slice, slice + 16, ... and
// the 16 slices meet through LDS in slice order, so the order of the
// additions is fixed and the result the same from run to run.
__global__ void __launch_bounds__(256)
    wino_filter_reduce_kernel(const float4* __restrict__ part,
                              float4* __restrict__ dw, unsigned n_vec,
                              int n_splits) {
  __shared__ float4 sums[16][16];
  const int e = threadIdx.x & 15, slice = threadIdx.x >> 4;
  const unsigned i = blockIdx.x * 16u + e;
  float4 a = make_float4(0.f, 0.f, 0.f, 0.f);
  if (i < n_vec) {
    for (int s = slice; s < n_splits; s += 16) {
      const float4 b = part[static_cast<size_t>(s) * n_vec + i];
      a = make_float4(a.x + b.x, a.y + b.y, a.z + b.z, a.w + b.w);
    }
  }
  sums[slice][e] = a;
  __syncthreads();
  if (slice == 0 && i < n_vec) {
    for (int q = 1; q < 16; ++q) {
      const float4 b = sums[q][e];
      a = make_float4(a.x + b.x, a.y + b.y, a.z + b.z, a.w + b.w);
    }
    dw[i] = a;
  }
}

// The same sum for a few splits: one float4 element per lane, the splits added
// in order (with two splits the kernel above leaves 14 of its 16 lane groups
// idle).
__global__ void __launch_bounds__(256)
    wino_filter_reduce_few_kernel(const float4* __restrict__ part,
                                  float4* __restrict__ dw, unsigned n_vec,
                                  int n_splits) {
  const unsigned i = blockIdx.x * 256u + threadIdx.x;
  if (i >= n_vec) return;
  float4 a = part[i];
  for (int s = 1; s < n_splits; ++s) {
    const float4 b = part[static_cast<size_t>(s) * n_vec + i];
    a = make_float4(a.x + b.x, a.y + b.y, a.z + b.z, a.w + b.w);
  }
  dw[i] = a;
}

struct FilterPlan {
  FilterGeom g;
  int splits;
};

FilterPlan plan_filter_backprop(const snn_hip_conv2d_params& p) {
  FilterPlan plan;
  FilterGeom& g = plan.g;
  g.batch = p.batch;
  g.in_rows = p.in_rows; g.in_cols = p.in_cols; g.channels = p.channels;
  g.out_rows = p.out_rows; g.out_cols = p.out_cols; g.features = p.features;
  g.pad_rows = p.pad_rows; g.pad_cols = p.pad_cols;
  g.tile_rows = ceil_div(p.out_rows, 2);
  g.tile_cols = ceil_div(p.out_cols, 2);
  g.n_tiles = p.batch * g.tile_rows * g.tile_cols;
  g.c_blocks = ceil_div(p.channels, kBC);
  g.k_blocks = ceil_div(p.features, kBK);
  // about one work-group per CU (256 on MI355X), each at least four steps
  const int blocks = g.c_blocks * g.k_blocks;
  int splits = max(1, 256 / blocks);
  splits = min(splits, max(1, g.n_tiles / (4 * kStepTiles)));
  int per = ceil_div(g.n_tiles, splits);
  per = ceil_div(per, kStepTiles) * kStepTiles;
  g.tiles_per_split = per;
  plan.splits = ceil_div(g.n_tiles, per);
  return plan;
}

}  // namespace

bool conv2d_winograd_filter_backprop_supports(const snn_hip_conv2d_params& p) {
  const size_t x = static_cast<size_t>(p.batch) * p.in_rows * p.in_cols *
                   p.channels;
  const size_t y = static_cast<size_t>(p.batch) * p.out_rows * p.out_cols *
                   p.features;
  return p.window_rows == 3 && p.window_cols == 3 && p.stride_rows == 1 &&
         p.stride_cols == 1 && p.pad_rows <= 2 && p.pad_cols <= 2 &&
         p.channels % 2 == 0 && p.features % 4 == 0 && p.channels >= 16 &&
         p.features >= 16 && x * sizeof(float) <= kMaxBufferBytes &&
         y * sizeof(float) <= kMaxBufferBytes;
}

size_t conv2d_winograd_filter_backprop_workspace(
    const snn_hip_conv2d_params& p) {
  const FilterPlan plan = plan_filter_backprop(p);
  if (plan.splits <= 1) return 0;
  return static_cast<size_t>(plan.splits) * 9 * p.channels * p.features;
}

int launch_conv2d_winograd_filter_backprop_f32(
    const float* x, const float* dy, float* dw, const snn_hip_conv2d_params& p,
    float* workspace, size_t workspace_elems, hipStream_t stream) {
  const FilterPlan plan = plan_filter_backprop(p);
  const FilterGeom& g = plan.g;
  const size_t dw_elems = static_cast<size_t>(9) * p.channels * p.features;
  const bool two_pass = plan.splits > 1;
  if (two_pass &&
      (workspace == nullptr || workspace_elems < plan.splits * dw_elems))
    return SNN_HIP_INSUFFICIENT_WORKSPACE;
  static const hipError_t attr = hipFuncSetAttribute(
      reinterpret_cast<const void*>(wino_filter_backprop_kernel),
      hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes);
  (void)attr;
  const unsigned n_groups =
      static_cast<unsigned>(plan.splits * g.c_blocks * g.k_blocks);
  const size_t x_elems = static_cast<size_t>(p.batch) * p.in_rows * p.in_cols *
                         p.channels;
  const size_t dy_elems = static_cast<size_t>(p.batch) * p.out_rows *
                          p.out_cols * p.features;
  KernelTimer timer(stream);
  hipLaunchKernelGGL(wino_filter_backprop_kernel, dim3(n_groups),
                     dim3(kThreadsWf), kLdsBytes, stream, x, dy,
                     two_pass ? workspace : dw, g,
                     static_cast<unsigned>(x_elems * 4),
                     static_cast<unsigned>(dy_elems * 4), n_groups, dw_elems);
  if (two_pass) {
    const unsigned n_vec = static_cast<unsigned>(dw_elems / 4);
    if (plan.splits <= 8)
      hipLaunchKernelGGL(wino_filter_reduce_few_kernel,
                         dim3(ceil_div(n_vec, 256u)), dim3(256), 0, stream,
                         reinterpret_cast<const float4*>(workspace),
                         reinterpret_cast<float4*>(dw), n_vec, plan.splits);
    else
      hipLaunchKernelGGL(wino_filter_reduce_kernel, dim3(ceil_div(n_vec, 16u)),
                         dim3(256), 0, stream,
                         reinterpret_cast<const float4*>(workspace),
                         reinterpret_cast<float4*>(dw), n_vec, plan.splits);
  }
  SNN_HIP_CHECK_LAUNCH();
  return SNN_HIP_OK;
}

}  // namespace snn
