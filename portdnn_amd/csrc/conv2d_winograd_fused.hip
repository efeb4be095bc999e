// Winograd F(2x2,3x3) convolution in one pass over the data (gfx950), forward
// and input backprop, fp32.
//
// Same mathematics as the three-stage chain in conv2d_winograd.hip, which
// follows portDNN's (include/portdnn/internal/conv2d/winograd/launch.h:63-264,
// src/conv2d/winograd/kernels/tiles_impl.h:70-240), but the transformed input
// V and the products M never reach HBM:
//
//   * a small kernel transforms the filter once per launch into U, stored in
//     the exact order the matrix instruction wants its B operand, so that the
//     main kernel fetches it with one contiguous 1 KiB wave load per
//     (xi, 32 features, 8 channels) straight into registers;
//   * a work-group owns 32 tiles (2x2 output pixels each) x 32 features and
//     walks the channels 16 at a time: every lane gathers one tile's 4x4
//     patch for a channel pair (zero-filling buffer loads for the padding),
//     applies Bt d B in registers and writes the 16 transformed values to
//     LDS as V[xi][tile][channel];
//   * wave w multiplies the four xi = 4w .. 4w+3 planes,
//     M[xi] (32 tiles x 32 features) += V[xi] (32 x 16) * U[xi] (16 x 32),
//     on v_mfma_f32_32x32x2_f32 (4 x 16 accumulator registers);
//   * at the end At m A is applied: along xi's column index inside each lane,
//     along its row index across the four waves through LDS, and the 2x2
//     output pixels are written with 16-byte stores (or float atomics when
//     the channel range is split across work-groups to fill the GPU).
//
// The multiplications done on the matrix cores are 16/36 of the direct
// algorithm's.
#include <cstdlib>

#include "gemm_tile.h"
#include "snn_kernels.h"

namespace snn {
namespace {

using gemm::comp;
using gemm::float16v;

constexpr int kTiles = 32;              // Winograd tiles per work-group
constexpr int kFeat = 32;               // features per work-group
constexpr int kChunk = 16;              // channels per LDS stage
constexpr unsigned kOob = 0x7FFFFFF0u;
constexpr size_t kMaxBufferBytes = 0x7FFFFFF0u;

typedef unsigned int uint4v __attribute__((ext_vector_type(4)));
typedef float float4v __attribute__((ext_vector_type(4)));

// The (tile block, feature block) units of a launch and how they are dealt
// to the 8 XCDs: xcd_m x xcd_f = 8.
struct UnitGrid {
  int n_mblocks, n_fblocks;
  int xcd_m, xcd_f;
};

struct FusedGeom {
  int in_rows, in_cols, in_ch;
  int out_rows, out_cols, out_ch;
  int pad_rows, pad_cols;
  int tile_rows, tile_cols;
  int n_tiles;
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
__device__ inline float4 operator+(float4 a, float4 b) {
  return make_float4(a.x + b.x, a.y + b.y, a.z + b.z, a.w + b.w);
}
__device__ inline float4 operator-(float4 a, float4 b) {
  return make_float4(a.x - b.x, a.y - b.y, a.z - b.z, a.w - b.w);
}

// U = G g Gt for four consecutive input channels of one output channel,
// written in B-operand order, 1 KiB per (xi, 32 features, group):
//   u[xi][co / 32][group][lane][ci % 4]
// with (group, lane) as the main kernel's matrix instruction wants them (see
// `order` below).
// For the input gradient g[r][s] = W[2-r][2-s][co][ci] (mirrored taps, channel
// and feature roles swapped).
// (The direction is a template parameter and each form loads all of its taps
// in one straight run before the arithmetic: with a run-time `backprop` the
// compiler put every tap's load in a branch of its own and let at most eight
// be in flight, five round trips to memory for a kernel that is nothing but
// latency on the small filters.)
template <bool BACKPROP>
__global__ void __launch_bounds__(256)
    wino_filter_pack_kernel(const float* __restrict__ w, float* __restrict__ u,
                            int channels, int features, int order) {
  const int cin = BACKPROP ? features : channels;
  const int cout = BACKPROP ? channels : features;
  const int idx = blockIdx.x * 256 + threadIdx.x;
  if (idx >= (cin / 4) * cout) return;
  const int co = idx % cout, cq = idx / cout;
  // g[t][r][s]: tap (r, s) of input channel 4 cq + t.  The four channels of
  // the quad are contiguous in W for the input gradient (W[2-r][2-s][co][ci]):
  // one 16-byte load per tap; forward they are a row of W apart.
  float g[4][3][3];
  if (BACKPROP) {
    float4 gq[3][3];
#pragma unroll
    for (int r = 0; r < 3; ++r)
#pragma unroll
      for (int s = 0; s < 3; ++s)
        gq[r][s] = *reinterpret_cast<const float4*>(
            w + ((static_cast<size_t>(2 - r) * 3 + (2 - s)) * channels + co) *
                    features + 4 * cq);
    __builtin_amdgcn_sched_barrier(0);  // every load before the first use
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int r = 0; r < 3; ++r)
#pragma unroll
        for (int s = 0; s < 3; ++s) g[t][r][s] = comp(gq[r][s], t);
  } else {
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int r = 0; r < 3; ++r)
#pragma unroll
        for (int s = 0; s < 3; ++s)
          g[t][r][s] = w[((static_cast<size_t>(r) * 3 + s) * channels + 4 * cq +
                          t) * features + co];
    __builtin_amdgcn_sched_barrier(0);
  }
  float uu[16][4];
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    float h[4][3];  // G g
#pragma unroll
    for (int s = 0; s < 3; ++s) {
      h[0][s] = g[t][0][s];
      h[1][s] = 0.5f * (g[t][0][s] + g[t][1][s] + g[t][2][s]);
      h[2][s] = 0.5f * (g[t][0][s] - g[t][1][s] + g[t][2][s]);
      h[3][s] = g[t][2][s];
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      uu[i * 4 + 0][t] = h[i][0];
      uu[i * 4 + 1][t] = 0.5f * (h[i][0] + h[i][1] + h[i][2]);
      uu[i * 4 + 2][t] = 0.5f * (h[i][0] - h[i][1] + h[i][2]);
      uu[i * 4 + 3][t] = h[i][2];
    }
  }
  const int fblocks = cout / kFeat;
  const int cgroups = cin / 8;
  // Order 0 (32x32x2 instruction): channel quad cq = ci / 4 is lane half
  // cq % 2 of group cq / 2 (a group is 8 consecutive channels), lane co % 32
  // within the half.  Order 1 (16x16x4 instruction, cin % 16 == 0): quad
  // cq = 4 c16 + q of feature co = 32 fb + 16 F + n is lane n + 16 q of group
  // 2 c16 + F (a group is 16 channels x 16 features).
  int group = cq >> 1;
  int lane = co % kFeat + 32 * (cq & 1);
  if (order == 1) {
    group = 2 * (cq >> 2) + ((co % kFeat) >> 4);
    lane = (co & 15) + 16 * (cq & 3);
  }
  const size_t base =
      ((static_cast<size_t>(co / kFeat) * cgroups + group) * 64 + lane) * 4;
  const size_t xi_stride = static_cast<size_t>(fblocks) * cgroups * 256;
#pragma unroll
  for (int xi = 0; xi < 16; ++xi) {
    *reinterpret_cast<float4*>(u + xi * xi_stride + base) =
        make_float4(uu[xi][0], uu[xi][1], uu[xi][2], uu[xi][3]);
  }
}

__global__ void __launch_bounds__(256)
    wino_zero_fill_kernel(float4* __restrict__ p, size_t n_vec) {
  const size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
  if (i < n_vec) p[i] = make_float4(0.f, 0.f, 0.f, 0.f);
}

// The main kernel: a work-group of 8 waves per (32 tiles, 32 features) unit in
// which waves 0-3 only multiply (wave w owns xi = 4w .. 4w+3, B operand
// straight from L2) and waves 4-7 only gather and transform the input.  V is double buffered in
// LDS, so the transform of chunk c+1 runs while chunk c is being multiplied
// and one barrier per chunk is enough.  V rows hold 16 floats without padding;
// the 16-byte group index is xor-ed with (tile / 2) % 4, which makes both the
// ds_read_b128 of the multiplying waves and the ds_write_b64 of the
// transforming waves conflict free.
constexpr int kVBuf = 16 * kTiles * kChunk;  // floats per V buffer (32 KiB)

template <bool ATOMIC>
__global__ void __launch_bounds__(512)
    __attribute__((amdgpu_waves_per_eu(4, 4)))
    wino_fused_kernel(const float* __restrict__ in,
                         const float* __restrict__ u, float* __restrict__ out,
                         FusedGeom g, unsigned in_bytes, unsigned u_bytes,
                         unsigned out_bytes, UnitGrid ug,
                         int chunks_per_split,
                         const float* __restrict__ bias, int relu) {
  __shared__ __align__(16) float lds_v[2 * kVBuf];
  __shared__ int lds_tile_off[kTiles];
  __shared__ int lds_tile_flags[kTiles];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  // Work-group b runs on XCD b % 8 (round-robin dispatch); XCD (a, c) of the
  // xcd_m x xcd_f arrangement owns one range of tile blocks and one range of
  // feature blocks, so its L2 holds only that slice of the input and of U.
  const int xcd = static_cast<int>(blockIdx.x & 7u);
  const int local = static_cast<int>(blockIdx.x >> 3);
  const int xa = xcd / ug.xcd_f, xc = xcd % ug.xcd_f;
  const int m_lo = xa * ug.n_mblocks / ug.xcd_m;
  const int m_hi = (xa + 1) * ug.n_mblocks / ug.xcd_m;
  const int f_lo = xc * ug.n_fblocks / ug.xcd_f;
  const int f_hi = (xc + 1) * ug.n_fblocks / ug.xcd_f;
  const int f_cnt = f_hi - f_lo;
  if (local >= (m_hi - m_lo) * f_cnt) return;  // whole group, before any barrier
  const unsigned n_fblocks = static_cast<unsigned>(ug.n_fblocks);
  const unsigned fb = static_cast<unsigned>(f_lo + local % f_cnt);
  const int mb = m_lo + local / f_cnt;
  const int n_chunks = g.in_ch / kChunk;
  const int chunk_begin = static_cast<int>(blockIdx.y) * chunks_per_split;
  const int chunk_end = min(n_chunks, chunk_begin + chunks_per_split);

  float16v acc[4];
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[j][v] = 0.f;

  if (wave >= 4) {
    // ---- gather + transform waves --------------------------------------
    const __amdgpu_buffer_rsrc_t in_rsrc = make_rsrc(in, in_bytes);
    const int ptid = tid - 256;
    const int tile_l = ptid >> 3, pair = ptid & 7;
    unsigned p_off[16];
    {
      const int tile = mb * kTiles + tile_l;
      const bool live = tile < g.n_tiles;
      const int tx = tile % g.tile_cols;
      const int t2 = tile / g.tile_cols;
      const int ty = t2 % g.tile_rows;
      const int n = t2 / g.tile_rows;
      const int y0 = 2 * ty - g.pad_rows, x0 = 2 * tx - g.pad_cols;
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int y = y0 + i, x = x0 + j;
          const bool ok = live && static_cast<unsigned>(y) <
                                      static_cast<unsigned>(g.in_rows) &&
                          static_cast<unsigned>(x) <
                              static_cast<unsigned>(g.in_cols);
          p_off[i * 4 + j] =
              ok ? static_cast<unsigned>(
                       (((n * g.in_rows + y) * g.in_cols + x) * g.in_ch +
                        2 * pair) * 4)
                 : kOob;
        }
      if (pair == 0) {
        lds_tile_off[tile_l] =
            live ? ((n * g.out_rows + 2 * ty) * g.out_cols + 2 * tx) *
                       g.out_ch * 4
                 : -1;
        lds_tile_flags[tile_l] = (2 * ty + 1 < g.out_rows ? 1 : 0) |
                                 (2 * tx + 1 < g.out_cols ? 2 : 0);
      }
    }
    float* const v_store =
        lds_v + tile_l * kChunk +
        4 * ((pair >> 1) ^ ((tile_l >> 1) & 3)) + 2 * (pair & 1);
    auto load_patch = [&](int chunk, float2 (&d)[16]) {
      const unsigned soff =
          static_cast<unsigned>(min(chunk, chunk_end - 1) * kChunk * 4);
#pragma unroll
      for (int q = 0; q < 16; ++q)
        d[q] = __builtin_bit_cast(
            float2,
            __builtin_amdgcn_raw_buffer_load_b64(in_rsrc, p_off[q], soff, 0));
    };
    auto transform_store = [&](const float2 (&d)[16], int buf) {
      float* const dst = v_store + buf * kVBuf;
      float2 t[4][4];  // Bt d
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        t[0][j] = d[0 * 4 + j] - d[2 * 4 + j];
        t[1][j] = d[1 * 4 + j] + d[2 * 4 + j];
        t[2][j] = d[2 * 4 + j] - d[1 * 4 + j];
        t[3][j] = d[1 * 4 + j] - d[3 * 4 + j];
      }
      constexpr int kXi = kTiles * kChunk;  // floats per xi plane
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        *reinterpret_cast<float2*>(dst + (i * 4 + 0) * kXi) = t[i][0] - t[i][2];
        *reinterpret_cast<float2*>(dst + (i * 4 + 1) * kXi) = t[i][1] + t[i][2];
        *reinterpret_cast<float2*>(dst + (i * 4 + 2) * kXi) = t[i][2] - t[i][1];
        *reinterpret_cast<float2*>(dst + (i * 4 + 3) * kXi) = t[i][1] - t[i][3];
      }
    };
    // Two patch register sets: the loads run two chunks ahead of the
    // transform that consumes them (chunk indices past the end re-read the
    // last chunk and are never stored).
    float2 d_even[16], d_odd[16];
    load_patch(chunk_begin, d_even);
    load_patch(chunk_begin + 1, d_odd);
    transform_store(d_even, 0);
    load_patch(chunk_begin + 2, d_even);
    __syncthreads();
    for (int c = chunk_begin; c < chunk_end; c += 2) {
      // chunk c is being multiplied from buffer 0
      if (c + 1 < chunk_end) transform_store(d_odd, 1);
      load_patch(c + 3, d_odd);
      __syncthreads();
      if (c + 1 >= chunk_end) break;
      // chunk c + 1 is being multiplied from buffer 1
      if (c + 2 < chunk_end) transform_store(d_even, 0);
      load_patch(c + 4, d_even);
      __syncthreads();
    }
  } else {
    // ---- multiplying waves ---------------------------------------------
    const __amdgpu_buffer_rsrc_t u_rsrc = make_rsrc(u, u_bytes);
    const unsigned u_lane = static_cast<unsigned>(lane) * 16u;
    const unsigned cgroups = static_cast<unsigned>(g.in_ch) / 8u;
    unsigned u_base[4];
#pragma unroll
    for (int j = 0; j < 4; ++j)
      u_base[j] = ((static_cast<unsigned>(4 * wave + j) * n_fblocks + fb) *
                   cgroups) * 1024u;
    auto load_b = [&](int cgroup, float4 (&b)[4]) {
#pragma unroll
      for (int j = 0; j < 4; ++j)
        b[j] = __builtin_bit_cast(
            float4, __builtin_amdgcn_raw_buffer_load_b128(
                        u_rsrc, u_lane,
                        u_base[j] + static_cast<unsigned>(cgroup) * 1024u, 0));
    };
    const int tile_r = lane & 31;
    const int swz = (tile_r >> 1) & 3;
    constexpr int kXi = kTiles * kChunk;
    const float* const a_base = lds_v + (4 * wave * kTiles + tile_r) * kChunk;
    const int a_grp0 = 4 * ((0 + (lane >> 5)) ^ swz);
    const int a_grp1 = 4 * ((2 + (lane >> 5)) ^ swz);
    auto mma_group = [&](const float* a_ptr, const float4 (&b)[4]) {
      float4 a[4];
#pragma unroll
      for (int j = 0; j < 4; ++j)
        a[j] = *reinterpret_cast<const float4*>(a_ptr + j * kXi);
#pragma unroll
      for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int j = 0; j < 4; ++j)
          acc[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(
              comp(a[j], t), comp(b[j], t), acc[j], 0, 0, 0);
    };
    float4 b_lo[4], b_hi[4];
    load_b(2 * chunk_begin, b_lo);
    load_b(2 * chunk_begin + 1, b_hi);
    __syncthreads();
    for (int c = chunk_begin; c < chunk_end; ++c) {
      const float* const a_buf = a_base + ((c - chunk_begin) & 1) * kVBuf;
      const int next = min(c + 1, chunk_end - 1);
      mma_group(a_buf + a_grp0, b_lo);
      load_b(2 * next, b_lo);
      mma_group(a_buf + a_grp1, b_hi);
      load_b(2 * next + 1, b_hi);
      __syncthreads();
    }
    // At m A along xi's column index, inside the lane.
    float* const s_base = lds_v + (wave * 2 * 16) * 64 + lane;
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      s_base[v * 64] = acc[0][v] + acc[1][v] + acc[2][v];
      s_base[(16 + v) * 64] = acc[1][v] - acc[2][v] - acc[3][v];
    }
  }
  __syncthreads();
  // Along xi's row index (across the multiplying waves); all 512 lanes write.
  const __amdgpu_buffer_rsrc_t out_rsrc = make_rsrc(out, out_bytes);
  const unsigned out_row_bytes =
      static_cast<unsigned>(g.out_cols) * g.out_ch * 4u;
  {
    const int b = tid >> 8;
    const int q = tid & 15;
    const int v = (tid >> 4) & 15;
    float4 s[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
      s[i] = *reinterpret_cast<const float4*>(
          lds_v + ((i * 2 + b) * 16 + v) * 64 + 4 * q);
    float4 y0 = s[0] + s[1] + s[2];
    float4 y1 = s[1] - s[2] - s[3];
    const int m = 8 * (v >> 2) + 4 * (q >> 3) + (v & 3);
    const int f = static_cast<int>(fb) * kFeat + 4 * (q & 7);
    if (!ATOMIC) {
      // Optional epilogue of the forward convolution: bias per feature, ReLU.
      if (bias != nullptr) {
        const float4 b4 = *reinterpret_cast<const float4*>(bias + f);
        y0 = y0 + b4;
        y1 = y1 + b4;
      }
      if (relu) {
        y0 = make_float4(fmaxf(y0.x, 0.f), fmaxf(y0.y, 0.f), fmaxf(y0.z, 0.f),
                         fmaxf(y0.w, 0.f));
        y1 = make_float4(fmaxf(y1.x, 0.f), fmaxf(y1.y, 0.f), fmaxf(y1.z, 0.f),
                         fmaxf(y1.w, 0.f));
      }
    }
    const int tile_off = lds_tile_off[m];
    const int flags = lds_tile_flags[m];
    const bool col_ok = tile_off >= 0 && (b == 0 || (flags & 2) != 0);
    const unsigned off0 =
        col_ok ? static_cast<unsigned>(tile_off) +
                     static_cast<unsigned>(b * g.out_ch + f) * 4u
               : kOob;
    const unsigned off1 =
        (col_ok && (flags & 1) != 0) ? off0 + out_row_bytes : kOob;
    if (ATOMIC) {
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        __builtin_amdgcn_raw_ptr_buffer_atomic_fadd_f32(
            comp(y0, e), out_rsrc, off0 + 4u * e, 0, 0);
        __builtin_amdgcn_raw_ptr_buffer_atomic_fadd_f32(
            comp(y1, e), out_rsrc, off1 + 4u * e, 0, 0);
      }
    } else {
      __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(uint4v, y0),
                                             out_rsrc, off0, 0, 0);
      __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(uint4v, y1),
                                             out_rsrc, off1, 0, 0);
    }
  }
}

// ---------------------------------------------------------------------------
// Persistent direct-to-LDS kernel: wino_fused_kernel's unit (32 tiles x 32
// features) and xi-row-per-wave multiplication, organised around what was
// measured on this GPU:
//
//   * Timestamps inside wino_fused_kernel: a unit's prologue (tile index
//     arithmetic, first gather from memory, first transform: 2.7 - 6.7 us)
//     and epilogue (1.3 us) are nearly half of its 14 us on a 64-channel
//     layer.  Here a work-group is persistent: it walks the units slot,
//     slot + G, ... of its XCD as one stream of 16-channel chunks, and the
//     next unit's index arithmetic and first loads happen while the current
//     one is being multiplied.
//   * The fp32 matrix instructions run on the vector ALUs: a wave of plain
//     v_add_f32 next to a wave streaming v_mfma_f32_32x32x2_f32 on the same
//     SIMD is issued nothing until that wave stops (whatever the waves' age
//     or priority).  Waves that only transform therefore take turns with the
//     multiplying waves instead of working alongside them.  Here no wave only
//     transforms: the additions sit in the multiplying wave's own
//     instruction stream.
//   * Per wave-level load of an L2-resident buffer: an 8-byte-per-lane gather
//     of 8 tiles x 64 bytes into registers costs 32 CU-cycles (16 B/clk), a
//     contiguous 16-byte register load 28, a 16-byte load that writes LDS
//     directly 13.5 (76 B/clk) whatever its address pattern.  64 register
//     gathers and 32 B loads per chunk are about 2900 CU-cycles of
//     vector-memory time per 2048 cycles of matrix instructions.  Here the
//     patches go from memory to LDS with buffer_load ... lds.
//
//   A work-group is 4 waves; wave w owns the xi = 4w .. 4w+3 planes and
//   fetches patch row w: 32 instructions per chunk and work-group, two 32 KiB
//   raw buffers, the chunk after the current one in flight.
//   raw[p][T][piece][t] is 16 bytes: pixel p of the 4x4 patch, tile 16 T + t,
//   channels 4 piece .. 4 piece + 3.  Each wave reads the two patch rows its
//   xi row combines (Bt d: d0 - d2, d1 + d2, d2 - d1, d1 - d3), applies the
//   column transform in registers and feeds the results to
//   v_mfma_f32_16x16x4_f32 as the A operand: lane (t, piece) holds tiles t and
//   16 + t, channels 4 piece .. 4 piece + 3 -- the order the gather's lanes
//   wrote the raw buffer in, so every lane reads back its own 16 bytes -- and
//   instruction e of a chunk reduces channels 4 q + e over the lane quarters q
//   (the filter pack orders U to match).  A unit is 2 x 2 blocks of 16 tiles x
//   16 features per xi plane (the 32x32x2 form of this kernel measured 1-2 %
//   slower on three of the four batch-32 ResNet layers, the same on the last).
//   The transformed input never exists in memory.  One barrier per chunk; at
//   the end of a unit At m A goes through the raw buffer that was multiplied
//   last (two more barriers).
//
// Two work-groups per CU (2 x 65 KiB LDS, up to 256 registers).  Requires an
// even number of chunks.
// ---------------------------------------------------------------------------
typedef __attribute__((address_space(3))) void* lds_void_ptr;
// The output is written once and not read again by the kernel: stream it
// (slc).  -1 ... -2 us on the 56x56x64 layer.
constexpr int kStoreAux = 2;
constexpr int kWaitVm8 = 0x0F78;  // s_waitcnt vmcnt(8)

__global__ void __launch_bounds__(256)
    __attribute__((amdgpu_waves_per_eu(2, 2)))
    wino_direct_kernel(const float* __restrict__ in,
                       const float* __restrict__ u, float* __restrict__ out,
                       FusedGeom g, unsigned in_bytes, unsigned u_bytes,
                       unsigned out_bytes, UnitGrid ug, float inv_tile_cols,
                       float inv_tile_rows, const float* __restrict__ bias,
                       int relu) {
  // Two raw buffers as two objects: the compiler then knows that the loads
  // that fill one do not touch the one being read, and does not make the
  // reads wait for them.
  __shared__ __align__(16) float lds_raw0[kVBuf];
  __shared__ __align__(16) float lds_raw1[kVBuf];
  __shared__ int lds_tile_off[2][kTiles];
  __shared__ int lds_tile_flags[2][kTiles];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int xcd = static_cast<int>(blockIdx.x & 7u);
  const int slot = static_cast<int>(blockIdx.x >> 3);
  const int stride = static_cast<int>(gridDim.x >> 3);
  const int xa = xcd / ug.xcd_f, xc = xcd % ug.xcd_f;
  const int m_lo = xa * ug.n_mblocks / ug.xcd_m;
  const int m_hi = (xa + 1) * ug.n_mblocks / ug.xcd_m;
  const int f_lo = xc * ug.n_fblocks / ug.xcd_f;
  const int f_hi = (xc + 1) * ug.n_fblocks / ug.xcd_f;
  const int f_cnt = f_hi - f_lo;
  const int n_local = (m_hi - m_lo) * f_cnt;
  if (slot >= n_local) return;  // whole group, before any barrier
  const int n_chunks = g.in_ch / kChunk;

  const __amdgpu_buffer_rsrc_t in_rsrc = make_rsrc(in, in_bytes);
  const __amdgpu_buffer_rsrc_t u_rsrc = make_rsrc(u, u_bytes);

  // ---- gather: lane (piece, t) of instruction (patch column pc, T) --------
  const int g_piece = lane >> 4, g_t = lane & 15;
  unsigned p_off[2][4];
  // Offsets of patch row `wave` of tiles t and 16 + t of unit `unit`, all out
  // of range (the loads then write zeros and fetch nothing) past the last
  // unit.  Wave 0 also notes where the unit's tiles go in the output.
  auto enter_unit = [&](int unit, int count) {
    const bool any = unit < n_local;
    const int mb = m_lo + unit / f_cnt;
#pragma unroll
    for (int T = 0; T < 2; ++T) {
      const int tile_l = 16 * T + g_t;
      const int tile = mb * kTiles + tile_l;
      const bool live = any && tile < g.n_tiles;
      // tile = (n * tile_rows + ty) * tile_cols + tx with tile < 2^23: the
      // float quotient is at most one off.
      int t2 = static_cast<int>(static_cast<float>(tile) * inv_tile_cols);
      int tx = tile - t2 * g.tile_cols;
      if (tx < 0) { tx += g.tile_cols; --t2; }
      if (tx >= g.tile_cols) { tx -= g.tile_cols; ++t2; }
      int n = static_cast<int>(static_cast<float>(t2) * inv_tile_rows);
      int ty = t2 - n * g.tile_rows;
      if (ty < 0) { ty += g.tile_rows; --n; }
      if (ty >= g.tile_rows) { ty -= g.tile_rows; ++n; }
      const int y = 2 * ty - g.pad_rows + wave;
      const int x0 = 2 * tx - g.pad_cols;
      const bool row_ok = live && static_cast<unsigned>(y) <
                                      static_cast<unsigned>(g.in_rows);
      const unsigned row_off =
          static_cast<unsigned>((n * g.in_rows + y) * g.in_cols) *
              static_cast<unsigned>(g.in_ch) * 4u +
          static_cast<unsigned>(g_piece) * 16u;
#pragma unroll
      for (int pc = 0; pc < 4; ++pc) {
        const int x = x0 + pc;
        const bool ok = row_ok && static_cast<unsigned>(x) <
                                      static_cast<unsigned>(g.in_cols);
        p_off[T][pc] =
            ok ? row_off + static_cast<unsigned>(x * g.in_ch) * 4u : kOob;
      }
      if (wave == 0 && g_piece == 0) {
        lds_tile_off[count & 1][tile_l] =
            live ? ((n * g.out_rows + 2 * ty) * g.out_cols + 2 * tx) *
                       g.out_ch * 4
                 : -1;
        lds_tile_flags[count & 1][tile_l] =
            (2 * ty + 1 < g.out_rows ? 1 : 0) |
            (2 * tx + 1 < g.out_cols ? 2 : 0);
      }
    }
  };
  // One of the eight loads of patch row `wave` of chunk `chunk` into a raw
  // buffer: instruction i = (pc, T) fills the 1 KiB block (4 wave + pc) * 2 + T.
  auto gather = [&](float* raw, int chunk, int i) {
    const unsigned soff = static_cast<unsigned>(chunk * kChunk * 4);
    char* const dst = reinterpret_cast<char*>(raw) + wave * 8 * 1024;
    __builtin_amdgcn_raw_ptr_buffer_load_lds(
        in_rsrc, (lds_void_ptr)(dst + i * 1024), 16, p_off[i & 1][i >> 1],
        soff, 0, 0);
  };

  // ---- multiply: lane (tile % 16, channel quad) --------------------------
  const unsigned n_fblocks = static_cast<unsigned>(ug.n_fblocks);
  const unsigned u_lane = static_cast<unsigned>(lane) * 16u;
  const unsigned cgroups = static_cast<unsigned>(g.in_ch) / 8u;
  // Byte offset of U[xi = 4 wave][feature block of `unit`][channel group 0].
  auto u_base_of = [&](int unit) {
    const unsigned fb = static_cast<unsigned>(f_lo + unit % f_cnt);
    return static_cast<unsigned>(__builtin_amdgcn_readfirstlane(
        ((static_cast<unsigned>(4 * wave) * n_fblocks + fb) * cgroups) *
        1024u));
  };
  const unsigned u_xi_stride = n_fblocks * cgroups * 1024u;
  auto load_b = [&](unsigned base, int cgroup, int j) {
    return __builtin_bit_cast(
        float4, __builtin_amdgcn_raw_buffer_load_b128(
                    u_rsrc, u_lane,
                    base + static_cast<unsigned>(j) * u_xi_stride +
                        static_cast<unsigned>(cgroup) * 1024u,
                    0));
  };
  // Bt d for xi row `wave`: patch rows ra and rb, t = d[ra] + sgn d[rb].
  const int ra = wave == 0 ? 0 : (wave == 2 ? 2 : 1);
  const int rb = wave == 0 ? 2 : (wave == 1 ? 2 : (wave == 2 ? 1 : 3));
  const float sgn = wave == 1 ? 1.f : -1.f;
  // Block (patch row r, column pc, tile half T) of a raw buffer is 1 KiB in
  // the order the gather's lanes wrote it -- tile 16 T + lane % 16, channel
  // quad lane / 16 -- which is the matrix instruction's operand order: every
  // lane reads its own 16 bytes.
  const int raw_a = ra * 8 * 256 + lane * 4;
  const int raw_b = rb * 8 * 256 + lane * 4;
  auto read_rows = [&](const float* raw, int T, float4 (&da)[4],
                       float4 (&db)[4]) {
#pragma unroll
    for (int pc = 0; pc < 4; ++pc) {
      da[pc] = *reinterpret_cast<const float4*>(raw + raw_a +
                                                (pc * 2 + T) * 256);
      db[pc] = *reinterpret_cast<const float4*>(raw + raw_b +
                                                (pc * 2 + T) * 256);
    }
  };
  auto fma4 = [&](const float4& x, const float4& y) {
    return make_float4(fmaf(y.x, sgn, x.x), fmaf(y.y, sgn, x.y),
                       fmaf(y.z, sgn, x.z), fmaf(y.w, sgn, x.w));
  };
  // (Bt d B) for this wave's xi row: a[j], four channels each.
  auto transform = [&](const float4 (&da)[4], const float4 (&db)[4],
                       float4 (&a)[4]) {
    const float4 t0 = fma4(da[0], db[0]), t1 = fma4(da[1], db[1]);
    const float4 t2 = fma4(da[2], db[2]), t3 = fma4(da[3], db[3]);
    a[0] = t0 - t2;
    a[1] = t1 + t2;
    a[2] = t2 - t1;
    a[3] = t1 - t3;
  };
  // acc[xi plane][tile half T][feature half F]: tiles 16 T + 4 (lane / 16)
  // + r, feature 16 F + lane % 16.
  float4v acc[4][2][2];
  // Four matrix instructions: reduction step e (channels 4 q + e over the
  // lane quarters q) of the four xi planes, one 16 x 16 block each.
  auto mma_group = [&](const float4 (&a)[4], const float4 (&b)[4], int e,
                       int T, int F) {
#pragma unroll
    for (int j = 0; j < 4; ++j)
      acc[j][T][F] = __builtin_amdgcn_mfma_f32_16x16x4f32(
          comp(a[j], e), comp(b[j], e), acc[j][T][F], 0, 0, 0);
  };
  // B operand: b0 for the first 16 features of the block, b1x / b1y in turn
  // for the second.
  float4 b0[4], b1x[4], b1y[4];
  // One chunk from `raw`: the first feature half against both tile halves,
  // then the second.  Every vector-memory instruction sits behind a group of
  // four matrix instructions (128 cycles of matrix work), so the texture
  // path takes them one at a time and the wave never stands at a full queue:
  // the eight gather loads of the next chunk of the stream (chunk g_chunk of
  // the unit the offsets are set for; into the other raw buffer, which every
  // wave finished reading before the barrier) behind the groups of the first
  // feature half, and behind those of the second the refills of b0 (used up
  // by then) and of the idle b1 for the chunk after (nb_base, nb_cg).  The
  // fences keep the compiler from collecting the loads in one place.
  auto step = [&](const float* raw, float* raw_next, int g_chunk,
                  float4 (&b1)[4], float4 (&b1_idle)[4], unsigned nb_base,
                  int nb_cg) {
    float4 da[4], db[4], a0[4], a1[4];
    read_rows(raw, 0, da, db);
    __builtin_amdgcn_sched_barrier(0);
    transform(da, db, a0);
    __builtin_amdgcn_sched_barrier(0);
    read_rows(raw, 1, da, db);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      mma_group(a0, b0, e, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
      gather(raw_next, g_chunk, e);
      __builtin_amdgcn_sched_barrier(0);
    }
    transform(da, db, a1);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      mma_group(a1, b0, e, 1, 0);
      __builtin_amdgcn_sched_barrier(0);
      gather(raw_next, g_chunk, 4 + e);
      __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      mma_group(a0, b1, e, 0, 1);
      __builtin_amdgcn_sched_barrier(0);
      b0[e] = load_b(nb_base, nb_cg, e);
      __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      mma_group(a1, b1, e, 1, 1);
      __builtin_amdgcn_sched_barrier(0);
      b1_idle[e] = load_b(nb_base, nb_cg + 1, e);
      __builtin_amdgcn_sched_barrier(0);
    }
    // The gather (eight loads, issued before the eight B loads) has landed.
    __builtin_amdgcn_s_waitcnt(kWaitVm8);
    __syncthreads();
  };

  // ---- start of the stream ------------------------------------------------
  enter_unit(slot, 0);
  unsigned u_base = u_base_of(slot);
#pragma unroll
  for (int i = 0; i < 8; ++i) gather(lds_raw0, 0, i);
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    b0[j] = load_b(u_base, 0, j);
    b1x[j] = load_b(u_base, 1, j);
  }
  __builtin_amdgcn_sched_barrier(0);
  __builtin_amdgcn_s_waitcnt(kWaitVm8);
  __syncthreads();

  const __amdgpu_buffer_rsrc_t out_rsrc = make_rsrc(out, out_bytes);
  const unsigned out_row_bytes =
      static_cast<unsigned>(g.out_cols) * g.out_ch * 4u;
  int count = 0;
  for (int unit = slot; unit < n_local; unit += stride, ++count) {
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int T = 0; T < 2; ++T)
#pragma unroll
        for (int F = 0; F < 2; ++F)
          acc[j][T][F] = float4v{0.f, 0.f, 0.f, 0.f};
    const int next_unit = unit + stride < n_local ? unit + stride : unit;
    const unsigned u_next = u_base_of(next_unit);
    // The unit's bias is fetched now: a load issued at the end of the unit
    // would have to wait for every load issued before it, the next unit's
    // first gather among them.
    const int fb = f_lo + unit % f_cnt;
    const int f = fb * kFeat + 4 * (tid & 7);
    float4 b4 = make_float4(0.f, 0.f, 0.f, 0.f);
    if (bias != nullptr) b4 = *reinterpret_cast<const float4*>(bias + f);
    for (int c = 0; c < n_chunks; c += 2) {
      step(lds_raw0, lds_raw1, c + 1, b1x, b1y, u_base, 2 * (c + 1));
      const bool last = c + 2 >= n_chunks;
      // The last chunk of a unit gathers the first one of the next unit.
      if (last) enter_unit(unit + stride, count + 1);
      step(lds_raw1, lds_raw0, last ? 0 : c + 2, b1y, b1x,
           last ? u_next : u_base, last ? 0 : 2 * (c + 2));
    }
    // At m A: along xi's column index inside the lane, into raw buffer 1
    // (every wave is past its reads of it; buffer 0 is being filled) ...
    // as s[xi row][output column ob][tile][feature], 32 floats per tile with
    // the two feature halves swapped for every other group of four tiles (so
    // that the lane quarters, four tiles apart, write different banks).
    {
      const int swz = 16 * ((lane >> 4) & 1);
      float* const s_base = lds_raw1 + wave * 2 * 1024 + (lane >> 4) * 4 * 32;
#pragma unroll
      for (int T = 0; T < 2; ++T)
#pragma unroll
        for (int F = 0; F < 2; ++F)
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const int at = (16 * T + r) * 32 + ((16 * F + (lane & 15)) ^ swz);
            s_base[at] = acc[0][T][F][r] + acc[1][T][F][r] + acc[2][T][F][r];
            s_base[1024 + at] =
                acc[1][T][F][r] - acc[2][T][F][r] - acc[3][T][F][r];
          }
    }
    __syncthreads();
    // ... then along its row index across the waves: thread (tile m, feature
    // quad tid % 8).
    const int m = tid >> 3;
    const int fq4 = (4 * (tid & 7)) ^ (16 * ((m >> 2) & 1));
    const int tile_off = lds_tile_off[count & 1][m];
    const int flags = lds_tile_flags[count & 1][m];
#pragma unroll
    for (int ob = 0; ob < 2; ++ob) {
      float4 s[4];
#pragma unroll
      for (int i = 0; i < 4; ++i)
        s[i] = *reinterpret_cast<const float4*>(
            lds_raw1 + ((i * 2 + ob) * 32 + m) * 32 + fq4);
      float4 y0 = s[0] + s[1] + s[2];
      float4 y1 = s[1] - s[2] - s[3];
      if (bias != nullptr) {
        y0 = y0 + b4;
        y1 = y1 + b4;
      }
      if (relu) {
        y0 = make_float4(fmaxf(y0.x, 0.f), fmaxf(y0.y, 0.f), fmaxf(y0.z, 0.f),
                         fmaxf(y0.w, 0.f));
        y1 = make_float4(fmaxf(y1.x, 0.f), fmaxf(y1.y, 0.f), fmaxf(y1.z, 0.f),
                         fmaxf(y1.w, 0.f));
      }
      const bool col_ok = tile_off >= 0 && (ob == 0 || (flags & 2) != 0);
      const unsigned off0 =
          col_ok ? static_cast<unsigned>(tile_off) +
                       static_cast<unsigned>(ob * g.out_ch + f) * 4u
                 : kOob;
      const unsigned off1 =
          (col_ok && (flags & 1) != 0) ? off0 + out_row_bytes : kOob;
      __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(uint4v, y0),
                                             out_rsrc, off0, 0, kStoreAux);
      __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(uint4v, y1),
                                             out_rsrc, off1, 0, kStoreAux);
    }
    __syncthreads();  // raw buffer 1 is free for the next unit's second chunk
    u_base = u_next;
  }
}

inline bool aligned16(const void* p) {
  return (reinterpret_cast<uintptr_t>(p) & 15u) == 0;
}

}  // namespace

bool conv2d_winograd_fused_supports(int direction,
                                    const snn_hip_conv2d_params& p) {
  if (!conv2d_winograd_supports(direction, p)) return false;
  const bool backprop = direction == SNN_HIP_INPUT_BACKPROP;
  const int in_ch = backprop ? p.features : p.channels;
  const int out_ch = backprop ? p.channels : p.features;
  const size_t x = static_cast<size_t>(p.batch) * p.in_rows * p.in_cols *
                   p.channels;
  const size_t y = static_cast<size_t>(p.batch) * p.out_rows * p.out_cols *
                   p.features;
  const size_t u = static_cast<size_t>(16) * p.channels * p.features;
  const size_t biggest = x > y ? (x > u ? x : u) : (y > u ? y : u);
  return in_ch % kChunk == 0 && out_ch % kFeat == 0 &&
         biggest * sizeof(float) <= kMaxBufferBytes;
}

int launch_conv2d_winograd_fused_f32(int direction, const float* input,
                                     const float* filter, float* output,
                                     const snn_hip_conv2d_params& p,
                                     float* workspace, size_t workspace_elems,
                                     hipStream_t stream,
                                     const LaunchOptions* epilogue) {
  const bool backprop = direction == SNN_HIP_INPUT_BACKPROP;
  FusedGeom g;
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
  g.n_tiles = p.batch * g.tile_rows * g.tile_cols;
  const size_t u_elems = static_cast<size_t>(16) * g.in_ch * g.out_ch;
  // Only U is stored, but the size contract stays the reference's minimum
  // (transformed filter plus one image of V and M, winograd/launch.h:237-261).
  const size_t per_image = static_cast<size_t>(16) * g.tile_rows *
                           g.tile_cols * (g.in_ch + g.out_ch);
  if (workspace == nullptr || workspace_elems < u_elems + per_image)
    return SNN_HIP_INSUFFICIENT_WORKSPACE;
  const bool prepare_only = epilogue != nullptr && epilogue->prepare_only;
  if (!aligned16(workspace) || (backprop && !aligned16(filter)) ||
      (!prepare_only && (!aligned16(input) || !aligned16(output))))
    return SNN_HIP_INVALID_PARAMETER;
  const size_t in_elems = static_cast<size_t>(p.batch) * g.in_rows *
                          g.in_cols * g.in_ch;
  const size_t out_elems = static_cast<size_t>(p.batch) * g.out_rows *
                           g.out_cols * g.out_ch;

  UnitGrid ug;
  ug.n_mblocks = ceil_div(g.n_tiles, kTiles);
  ug.n_fblocks = g.out_ch / kFeat;
  const unsigned n_units = static_cast<unsigned>(ug.n_mblocks) * ug.n_fblocks;
  // Each XCD has its own L2: with the XCDs arranged xcd_m x xcd_f over (tile
  // blocks, feature blocks), U is fetched from memory xcd_m times and the
  // input xcd_f times.  Take the arrangement with the least traffic that
  // still gives every XCD work.
  ug.xcd_m = 8;
  ug.xcd_f = 1;
  {
    double best = -1.0;
    for (int xf = 1; xf <= 8; xf *= 2) {
      const int xm = 8 / xf;
      if (xf > ug.n_fblocks || (xm > ug.n_mblocks && xm > 1)) continue;
      const double traffic = static_cast<double>(u_elems) * xm +
                             static_cast<double>(in_elems) * xf;
      if (best < 0.0 || traffic < best) {
        best = traffic;
        ug.xcd_m = xm;
        ug.xcd_f = xf;
      }
    }
  }
  if (const char* tune = SNN_TUNING_ENV("SNN_HIP_WINO_XCDF")) {
    const int xf = std::atoi(tune);
    if (xf == 1 || xf == 2 || xf == 4 || xf == 8) {
      ug.xcd_f = xf;
      ug.xcd_m = 8 / xf;
    }
  }
  const unsigned grid_x =
      8u * static_cast<unsigned>(ceil_div(ug.n_mblocks, ug.xcd_m)) *
      static_cast<unsigned>(ceil_div(ug.n_fblocks, ug.xcd_f));
  const int n_chunks = g.in_ch / kChunk;
  // Splitting the channel range across work-groups costs a zero fill and
  // float atomics on every output (measured: slower than leaving CUs idle as
  // soon as there are a few hundred units), so it is kept for launches that
  // would otherwise occupy only a fraction of the GPU.
  constexpr unsigned kFewUnits = 128;
  constexpr unsigned kTargetGroups = 512;
  constexpr int kMinChunks = 4;
  int splits = 1;
  const bool deterministic = epilogue != nullptr && epilogue->deterministic;
  if (n_units < kFewUnits && !deterministic)
    splits = static_cast<int>(ceil_div(kTargetGroups, n_units));
  splits = max(1, min(splits, n_chunks / kMinChunks));
  if (const char* tune = SNN_TUNING_ENV("SNN_HIP_WINO")) {
    if (tune[0] != 0) splits = max(1, min(std::atoi(tune), n_chunks));
  }
  const int per_split = ceil_div(n_chunks, splits);
  splits = ceil_div(n_chunks, per_split);

  const unsigned in_bytes = static_cast<unsigned>(in_elems * 4);
  const unsigned u_bytes = static_cast<unsigned>(u_elems * 4);
  const unsigned out_bytes = static_cast<unsigned>(out_elems * 4);
  // The persistent kernel takes every launch that is not split and has an
  // even number of chunks; it wants U in the 16x16x4 instruction's order.
  const bool persistent = splits == 1 && n_chunks % 2 == 0;
  const int pack_order = persistent ? 1 : 0;
  // The transformed filter depends on the filter and on this launch plan
  // only.  A caller that runs many launches with one filter may have it
  // written once (prepare_only) and then launch with filter_prepared, which
  // trusts what the workspace holds.
  const bool prepared = epilogue != nullptr && epilogue->filter_prepared;
  if (!prepared)
    hipLaunchKernelGGL(backprop ? wino_filter_pack_kernel<true>
                                : wino_filter_pack_kernel<false>,
                       dim3(ceil_div((g.in_ch / 4) * g.out_ch, 256)),
                       dim3(256), 0, stream, filter, workspace, p.channels,
                       p.features, pack_order);
  if (epilogue != nullptr && epilogue->prepare_only) {
    SNN_HIP_CHECK_LAUNCH();
    return SNN_HIP_OK;
  }
  if (splits > 1) {
    const size_t n_vec = out_elems / 4;  // out_ch % 32 == 0
    hipLaunchKernelGGL(wino_zero_fill_kernel,
                       dim3(static_cast<unsigned>(ceil_div(n_vec, size_t{256}))),
                       dim3(256), 0, stream, reinterpret_cast<float4*>(output),
                       n_vec);
    KernelTimer timer(stream);
    hipLaunchKernelGGL(wino_fused_kernel<true>, dim3(grid_x, splits),
                       dim3(512), 0, stream, input, workspace, output, g,
                       in_bytes, u_bytes, out_bytes, ug, per_split,
                       static_cast<const float*>(nullptr), 0);
  } else if (persistent) {
    // The bias vector is read 16 bytes at a time.
    const bool fuse = epilogue != nullptr && epilogue->wanted() && !backprop &&
                      (epilogue->bias == nullptr || aligned16(epilogue->bias));
    // Persistent work-groups, two per CU (32 CUs per XCD), fewer when an XCD
    // has fewer units.
    const unsigned per_xcd = grid_x / 8u;
    const unsigned groups_per_xcd = per_xcd < 64u ? per_xcd : 64u;
    KernelTimer timer(stream);
    hipLaunchKernelGGL(wino_direct_kernel, dim3(8u * groups_per_xcd),
                       dim3(256), 0, stream, input, workspace, output, g,
                       in_bytes, u_bytes, out_bytes, ug,
                       1.0f / static_cast<float>(g.tile_cols),
                       1.0f / static_cast<float>(g.tile_rows),
                       fuse ? epilogue->bias : nullptr,
                       fuse && epilogue->relu ? 1 : 0);
    if (fuse && epilogue->applied != nullptr) *epilogue->applied = true;
  } else {
    // The bias vector is read 16 bytes at a time.
    const bool fuse = epilogue != nullptr && epilogue->wanted() && !backprop &&
                      (epilogue->bias == nullptr || aligned16(epilogue->bias));
    KernelTimer timer(stream);
    hipLaunchKernelGGL(wino_fused_kernel<false>, dim3(grid_x, 1), dim3(512),
                       0, stream, input, workspace, output, g, in_bytes,
                       u_bytes, out_bytes, ug, per_split,
                       fuse ? epilogue->bias : nullptr,
                       fuse && epilogue->relu ? 1 : 0);
    if (fuse && epilogue->applied != nullptr) *epilogue->applied = true;
  }
  SNN_HIP_CHECK_LAUNCH();
  return SNN_HIP_OK;
}

}  // namespace snn
