// Dense convolution as an implicit GEMM on MFMA (gfx950).
//
// This is the MI355X counterpart of portDNN's Tiled kernels
// (src/conv2d/tiled/kernels.h:57-395) and of its Im2col + matmul chain
// (include/portdnn/internal/conv2d/im2col.h:43-327, src/conv2d/im2col/,
// src/matmul/kernels.h): the im2col matrix is never written to memory -- each
// work-group gathers the rows it needs straight into its LDS tile -- and the
// contraction runs on v_mfma_f32_32x32x2_f32.
//
//   forward          Y[m][k]  = sum_q A[m][q] * W[q][k]
//                    m = (n, oy, ox), q = (r, s, c);  A gathered from X,
//                    W is the HWCF filter read as a [R*S*C][K] matrix.
//   input backprop   dX[m][c] = sum_q A[m][q] * Wt[q][c]
//                    m = (n, y, x),  q = (r, s, k);   A gathered from dY at
//                    ((y + pad - r) / stride, (x + pad - s) / stride) where
//                    that divides, Wt[q][c] = W[r][s][c][k] (k contiguous).
//   filter backprop  dW[q][k] = sum_m A[m][q] * dY[m][k]
//                    reduction over every output pixel; the reduction is split
//                    across work-groups and combined with float atomics.
#include <cstdio>
#include <cstdlib>

#include "gemm_tile.h"
#include "snn_kernels.h"

namespace snn {
namespace {

using namespace gemm;

// Geometry of the gather.  "P" is the pixel grid the GEMM rows enumerate
// (output pixels for forward, input pixels for input backprop); "src" is the
// tensor the A operand is gathered from.
struct Gather {
  int batch;
  int p_rows, p_cols;      // pixel grid of the GEMM rows
  int src_rows, src_cols;  // spatial size of the gathered tensor
  int src_ch;              // channels of the gathered tensor (contiguous)
  int win_rows, win_cols;
  int step_rows, step_cols;  // pixel -> source coordinate multiplier
  int off_rows, off_cols;    // added to pixel * step
  int tap_sign;              // +1 forward (src = base + tap), -1 input backprop
  int div_rows, div_cols;    // source coordinate divisor (input backprop stride)
  int m_total;               // batch * p_rows * p_cols
  int k_total;               // win_rows * win_cols * src_ch
  int n_total;               // GEMM columns
  // Independent problems of the same shape (blockIdx.z): element strides
  // between their operands.  All zero for a convolution.
  int z_src, z_wgt, z_dst;
};

// Buffer addressing: loads go through raw buffer descriptors so that an
// out-of-range byte offset returns zeros.  Padding taps, rows past the last
// pixel and the ragged end of the reduction all become "offset = kOob" with
// no branch and no select on the loaded data.
typedef unsigned int uint4v __attribute__((ext_vector_type(4)));
constexpr unsigned kOob = 0x7FFFFFF0u;       // beyond any accepted tensor
constexpr size_t kMaxBufferBytes = 0x7FFFFFF0u;

__device__ inline __amdgpu_buffer_rsrc_t make_rsrc(const void* p,
                                                   unsigned bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, bytes,
                                           0x00020000);
}
__device__ inline float4 buffer_load4(__amdgpu_buffer_rsrc_t r, unsigned off) {
  const uint4v v = __builtin_amdgcn_raw_buffer_load_b128(r, off, 0, 0);
  return __builtin_bit_cast(float4, v);
}
// Four consecutive elements of storage type T at byte offset `off`, as floats
// (half-precision tensors are multiplied on the fp32 matrix instructions, so
// every product and sum is exactly what an f16 instruction with fp32
// accumulation would give).
template <typename T>
__device__ inline float4 buffer_load4_as_float(__amdgpu_buffer_rsrc_t r,
                                               unsigned off) {
  if constexpr (sizeof(T) == 4) {
    return buffer_load4(r, off);
  } else {
    typedef _Float16 half4 __attribute__((ext_vector_type(4)));
    typedef unsigned int uint2v __attribute__((ext_vector_type(2)));
    const uint2v v = __builtin_amdgcn_raw_buffer_load_b64(r, off, 0, 0);
    const half4 h = __builtin_bit_cast(half4, v);
    return make_float4(static_cast<float>(h.x), static_cast<float>(h.y),
                       static_cast<float>(h.z), static_cast<float>(h.w));
  }
}

// SCALAR_A: the gathered tensor's channel count is not a multiple of 4 (e.g.
// the 3-channel stem), so four consecutive reduction indices are not four
// consecutive floats of one tap; each is located and loaded on its own.
template <int BM, int BN, int WM, int WN, bool B_K_INNER, bool STRIDED,
          bool ATOMIC, bool SCALAR_A = false, typename T = float>
__global__ void __launch_bounds__(kThreads)
    conv_igemm_kernel(const T* __restrict__ src, const T* __restrict__ wgt,
                      T* __restrict__ dst, Gather g, unsigned src_bytes,
                      unsigned wgt_bytes, unsigned n_tiles_n, unsigned n_tiles,
                      int chunks_per_split) {
  static_assert(WM * WN == 4, "four waves per work-group");
  static_assert(sizeof(T) == 4 || (!ATOMIC && !SCALAR_A),
                "half-precision tensors: plain stores, vector gather");
  constexpr unsigned kEsz = sizeof(T);
  constexpr int WTM = BM / WM, WTN = BN / WN;  // wave tile
  constexpr int TM = WTM / 32, TN = WTN / 32;  // MFMA blocks per wave
  static_assert(TM >= 1 && TN >= 1, "wave tile must hold a 32x32 block");
  static_assert(!(SCALAR_A && STRIDED), "scalar gather is forward-style only");
  constexpr int A_FLOATS = k_inner_floats(BM);
  constexpr int B_FLOATS =
      B_K_INNER ? k_inner_floats(BN) : row_inner_floats(BN);
  constexpr int STAGE_FLOATS = A_FLOATS + B_FLOATS;
  extern __shared__ __align__(16) float lds[];  // two stages of [A tile | B tile]

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wave_m = wave / WN, wave_n = wave % WN;

  const unsigned tile = xcd_remap(blockIdx.x, n_tiles);
  const int m0 = static_cast<int>(tile / n_tiles_n) * BM;
  const int n0 = static_cast<int>(tile % n_tiles_n) * BN;
  // reduction range of this work-group (blockIdx.y = split index)
  const int n_chunks_total = (g.k_total + kBK - 1) / kBK;
  const int chunk_begin = blockIdx.y * chunks_per_split;
  const int n_chunks = min(chunks_per_split, n_chunks_total - chunk_begin);
  const int q_begin = chunk_begin * kBK;

  const __amdgpu_buffer_rsrc_t src_rsrc = make_rsrc(src, src_bytes);
  const __amdgpu_buffer_rsrc_t wgt_rsrc = make_rsrc(wgt, wgt_bytes);

  // ---- A gather bookkeeping: this lane copies chunk column `a_cc` (4 floats
  // at reduction offset 4 * a_cc) of tile rows a_r0 + 32 * i.
  constexpr int A_ROWS_PER_THREAD = BM / 32;
  const int a_cc = tid & 7;
  const int a_r0 = tid >> 3;
  int a_off[A_ROWS_PER_THREAD];  // element offset of (n, iy0, ix0, channel 0)
  int a_iy0[A_ROWS_PER_THREAD], a_ix0[A_ROWS_PER_THREAD];
#pragma unroll
  for (int i = 0; i < A_ROWS_PER_THREAD; ++i) {
    const int m = m0 + a_r0 + 32 * i;
    if (m < g.m_total) {
      const int px = m % g.p_cols;
      const int t = m / g.p_cols;
      const int py = t % g.p_rows;
      const int n = t / g.p_rows;
      a_iy0[i] = py * g.step_rows + g.off_rows;
      a_ix0[i] = px * g.step_cols + g.off_cols;
      a_off[i] = n * g.src_rows * g.src_cols * g.src_ch;
      if (!STRIDED) {
        a_off[i] += (a_iy0[i] * g.src_cols + a_ix0[i]) * g.src_ch;
      }
    } else {
      a_iy0[i] = -(1 << 28);  // never in range
      a_ix0[i] = 0;
      a_off[i] = 0;
    }
  }
  // (tap row, tap col, channel) of this lane's chunk; advanced by BK per step
  int a_c, a_s, a_r;
  {
    const int q = q_begin + 4 * a_cc;
    const int tap = q / g.src_ch;
    a_c = q - tap * g.src_ch;
    a_r = tap / g.win_cols;
    a_s = tap - a_r * g.win_cols;
  }

  // ---- B copy bookkeeping
  constexpr int B_VEC_PER_ROW = B_K_INNER ? kBK / 4 : BN / 4;
  constexpr int B_ROWS_PER_PASS = kThreads / B_VEC_PER_ROW;
  constexpr int B_PASSES = (B_K_INNER ? BN : kBK) / B_ROWS_PER_PASS;
  const int b_vec = tid % B_VEC_PER_ROW;
  const int b_row0 = tid / B_VEC_PER_ROW;

  float4 a_reg[A_ROWS_PER_THREAD];
  float4 b_reg[B_PASSES];

  int a_q = q_begin + 4 * a_cc;  // SCALAR_A: first reduction index of the lane
  auto load_a_scalar = [&]() {
    // (tap row, tap col, channel) of the four indices, by carry from the first
    int r = a_r, sc = a_s, c = a_c;
    int tap_off[4], tr[4], ts[4];
    bool q_ok[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      q_ok[e] = a_q + e < g.k_total;
      tr[e] = r;
      ts[e] = sc;
      tap_off[e] = (r * g.src_cols + sc) * g.src_ch + c;
      if (++c == g.src_ch) {
        c = 0;
        if (++sc == g.win_cols) { sc = 0; ++r; }
      }
    }
#pragma unroll
    for (int i = 0; i < A_ROWS_PER_THREAD; ++i) {
      float v[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int iy = a_iy0[i] + tr[e];
        const int ix = a_ix0[i] + ts[e];
        const bool ok =
            q_ok[e] &
            (static_cast<unsigned>(iy) < static_cast<unsigned>(g.src_rows)) &
            (static_cast<unsigned>(ix) < static_cast<unsigned>(g.src_cols));
        v[e] = __builtin_bit_cast(
            float, __builtin_amdgcn_raw_buffer_load_b32(
                       src_rsrc,
                       ok ? static_cast<unsigned>(a_off[i] + tap_off[e]) * 4u
                          : kOob,
                       0, 0));
      }
      a_reg[i] = make_float4(v[0], v[1], v[2], v[3]);
    }
  };
  auto load_a = [&]() {
    if (SCALAR_A) {
      load_a_scalar();
      return;
    }
    const bool tap_ok = a_r < g.win_rows;
    // offset of this lane's tap relative to (iy0, ix0)
    const int tap_off =
        g.tap_sign * (a_r * g.src_cols + a_s) * g.src_ch + a_c;
#pragma unroll
    for (int i = 0; i < A_ROWS_PER_THREAD; ++i) {
      int iy = a_iy0[i] + g.tap_sign * a_r;
      int ix = a_ix0[i] + g.tap_sign * a_s;
      bool ok = tap_ok;
      int off;
      if (STRIDED) {
        ok = ok & (iy >= 0) & (ix >= 0) & (iy % g.div_rows == 0) &
             (ix % g.div_cols == 0);
        iy /= g.div_rows;
        ix /= g.div_cols;
        off = a_off[i] + (iy * g.src_cols + ix) * g.src_ch + a_c;
      } else {
        off = a_off[i] + tap_off;
      }
      // bitwise, not short-circuit: no branches in the gather
      ok = ok &
           (static_cast<unsigned>(iy) < static_cast<unsigned>(g.src_rows)) &
           (static_cast<unsigned>(ix) < static_cast<unsigned>(g.src_cols));
      a_reg[i] = buffer_load4_as_float<T>(
          src_rsrc, ok ? static_cast<unsigned>(off) * kEsz : kOob);
    }
  };
  auto advance_a = [&]() {
    if (SCALAR_A) {
      a_q += kBK;
      const int tap = a_q / g.src_ch;
      a_c = a_q - tap * g.src_ch;
      a_r = tap / g.win_cols;
      a_s = tap - a_r * g.win_cols;
      return;
    }
    a_c += kBK;
    while (a_c >= g.src_ch) {
      a_c -= g.src_ch;
      if (++a_s == g.win_cols) { a_s = 0; ++a_r; }
    }
  };
  auto load_b = [&](int k0) {
#pragma unroll
    for (int i = 0; i < B_PASSES; ++i) {
      unsigned off = kOob;
      if (B_K_INNER) {
        // Wt[q][col]: element (col, q) lives at wgt[(tap * n_total + col) *
        // src_ch + kk] with q = tap * src_ch + kk; rows of the LDS tile are
        // GEMM columns, 4 consecutive q per lane.
        const int col = n0 + b_row0 + B_ROWS_PER_PASS * i;
        const int q = k0 + 4 * b_vec;
        if (col < g.n_total && q < g.k_total) {
          const int tap = q / g.src_ch;
          const int kk = q - tap * g.src_ch;
          off = static_cast<unsigned>((tap * g.n_total + col) * g.src_ch + kk) *
                kEsz;
        }
      } else {
        // W[q][col], col contiguous; q >= k_total is past the end of the
        // buffer and reads zeros by itself.
        const int q = k0 + b_row0 + B_ROWS_PER_PASS * i;
        const int col = n0 + 4 * b_vec;
        if (col < g.n_total)
          off = static_cast<unsigned>(q * g.n_total + col) * kEsz;
      }
      b_reg[i] = buffer_load4_as_float<T>(wgt_rsrc, off);
    }
  };
  auto store_tiles = [&](int stage) {
#pragma unroll
    for (int i = 0; i < A_ROWS_PER_THREAD; ++i) {
      *reinterpret_cast<float4*>(lds + stage * STAGE_FLOATS +
                                 (a_r0 + 32 * i) * (kBK + kPad) + 4 * a_cc) =
          a_reg[i];
    }
#pragma unroll
    for (int i = 0; i < B_PASSES; ++i) {
      const int row = b_row0 + B_ROWS_PER_PASS * i;
      float* b_tile = lds + stage * STAGE_FLOATS + A_FLOATS;
      float* p = B_K_INNER ? b_tile + row * (kBK + kPad) + 4 * b_vec
                           : b_tile + row * (BN + kPad) + 4 * b_vec;
      *reinterpret_cast<float4*>(p) = b_reg[i];
    }
  };

  float16v acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  load_a();
  load_b(q_begin);
  advance_a();
  store_tiles(0);
  __syncthreads();
  for (int it = 0; it < n_chunks; ++it) {
    const int stage = it & 1;
    const bool more = it + 1 < n_chunks;
    if (more) {
      load_a();
      load_b(q_begin + (it + 1) * kBK);
      advance_a();
    }
    mma_chunk<TM, TN, true, B_K_INNER, BM, BN>(
        lds + stage * STAGE_FLOATS, lds + stage * STAGE_FLOATS + A_FLOATS,
        wave_m * WTM, wave_n * WTN, lane, acc);
    if (more) store_tiles(stage ^ 1);
    __syncthreads();
  }

  // ---- epilogue: accumulator (row = 8*(v/4) + 4*(lane/32) + v%4, col =
  // lane%32) -> dst[m][col]
  const int col_l = lane & 31;
  const int row_l = 4 * (lane >> 5);
#pragma unroll
  for (int i = 0; i < TM; ++i) {
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int col = n0 + wave_n * WTN + 32 * j + col_l;
      if (col >= g.n_total) continue;
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int m = m0 + wave_m * WTM + 32 * i + 8 * (v >> 2) + row_l + (v & 3);
        if (m < g.m_total) {
          T* o = dst + static_cast<size_t>(m) * g.n_total + col;
          if constexpr (ATOMIC)
            unsafeAtomicAdd(o, acc[i][j][v]);
          else
            *o = static_cast<T>(acc[i][j][v]);
        }
      }
    }
  }
}

// ---------------------------------------------------------------------------
// Fast path.  The gather of the generic kernel spends dozens of integer
// vector instructions (multiplies, divisions by the channel count) per chunk
// and lane; this kernel keeps per-chunk vector work to three instructions per
// gathered row and nothing else:
//   * src_ch % 32 == 0, so a 32-wide reduction chunk lies inside one filter
//     tap and the tap / channel bookkeeping is wave-uniform (scalar ALU);
//   * per-row validity of every tap is a precomputed 32-bit mask; an invalid
//     tap sets bit 31 of the buffer offset, which the descriptor's range
//     check turns into a zero fill;
//   * weight and output accesses use a per-lane constant offset plus a scalar
//     offset operand, LDS addresses are constants plus immediates (the chunk
//     loop is unrolled by the two LDS stages).
//
// EPI: the forward convolution's optional epilogue, out = act(acc +
// bias[feature]), applied to the accumulators before they are stored.
template <int BM, int BN, int WM, int WN, bool B_K_INNER, bool ATOMIC,
          bool EPI = false>
__global__ void __launch_bounds__(kThreads)
    conv_igemm_fast_kernel(const float* __restrict__ src,
                           const float* __restrict__ wgt,
                           float* __restrict__ dst, Gather g,
                           unsigned src_bytes, unsigned wgt_bytes,
                           unsigned dst_bytes, unsigned n_tiles_n,
                           unsigned n_tiles, int chunks_per_split,
                           const float* __restrict__ bias = nullptr,
                           int relu = 0) {
  static_assert(!(EPI && ATOMIC), "partial sums cannot take the epilogue");
  static_assert(WM * WN == 4, "four waves per work-group");
  constexpr int WTM = BM / WM, WTN = BN / WN;
  constexpr int TM = WTM / 32, TN = WTN / 32;
  constexpr int A_FLOATS = k_inner_floats(BM);
  constexpr int B_FLOATS =
      B_K_INNER ? k_inner_floats(BN) : row_inner_floats(BN);
  constexpr int STAGE_FLOATS = A_FLOATS + B_FLOATS;
  extern __shared__ __align__(16) float lds[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wave_m = wave / WN, wave_n = wave % WN;

  const int chunks_per_tap = g.src_ch / kBK;
  const int n_chunks_total = g.win_rows * g.win_cols * chunks_per_tap;
  const int chunk_begin = blockIdx.y * chunks_per_split;
  const int n_chunks = min(chunks_per_split, n_chunks_total - chunk_begin);

  src += static_cast<size_t>(blockIdx.z) * g.z_src;
  wgt += static_cast<size_t>(blockIdx.z) * g.z_wgt;
  dst += static_cast<size_t>(blockIdx.z) * g.z_dst;
  const __amdgpu_buffer_rsrc_t src_rsrc = make_rsrc(src, src_bytes);
  const __amdgpu_buffer_rsrc_t wgt_rsrc = make_rsrc(wgt, wgt_bytes);
  const __amdgpu_buffer_rsrc_t dst_rsrc = make_rsrc(dst, dst_bytes);

  // A work-group walks the tiles blockIdx.x, blockIdx.x + gridDim.x, ... (the
  // launcher starts no more work-groups than fit on the GPU at once), so the
  // hardware does not have to retire and dispatch a work-group per tile and
  // the first loads of a tile are in flight while the previous one is stored.

  // ---- A gather: lane copies 16 bytes at chunk column a_cc of tile rows
  // a_r0 + 32 * i.  a_voff = byte offset of (n, iy0, ix0, 4 * a_cc) in two's
  // complement (it may lie before the tensor for border pixels; adding a
  // valid tap's offset brings it back in range).
  constexpr int A_PASSES = BM / 32;
  const int a_cc = tid & 7;
  const int a_r0 = tid >> 3;
  unsigned a_voff[A_PASSES];
  unsigned a_inval[A_PASSES];  // bit t set: filter tap t is padding
  // A 1x1 window at stride 1 without padding reads row m of the source as it
  // is (plain GEMM): no pixel decomposition, no tap masks.  The test is
  // uniform, so a launch pays for one of the two set-ups only.
  const bool plain_rows = g.win_rows == 1 && g.win_cols == 1 &&
                          g.step_rows == 1 && g.step_cols == 1 &&
                          g.off_rows == 0 && g.off_cols == 0 &&
                          g.src_rows == g.p_rows && g.src_cols == g.p_cols;

  // ---- B copy: per-lane constant offsets, scalar chunk offsets
  constexpr int B_VEC_PER_ROW = B_K_INNER ? kBK / 4 : BN / 4;
  constexpr int B_ROWS_PER_PASS = kThreads / B_VEC_PER_ROW;
  constexpr int B_PASSES = (B_K_INNER ? BN : kBK) / B_ROWS_PER_PASS;
  const int b_vec = tid % B_VEC_PER_ROW;
  const int b_row0 = tid / B_VEC_PER_ROW;
  unsigned b_voff[B_K_INNER ? B_PASSES : 1];
  // scalar byte strides
  const unsigned b_pass_stride =
      static_cast<unsigned>(B_ROWS_PER_PASS * g.n_total) * 4u;  // NN only
  const unsigned b_tap_stride =
      static_cast<unsigned>(g.n_total * g.src_ch) * 4u;  // K-inner only

  // wave-uniform reduction position: tap index, its (row, col), channel base
  int tap, c0, tap_r, tap_c, chunk;
  const int chunk_end = chunk_begin + n_chunks;

  // Per-tile set-up of the load side: addresses of tile `logical` and the
  // reduction position back at the start of this work-group's chunk range.
  auto setup_tile = [&](unsigned logical, int* m0_out, int* n0_out) {
    const unsigned tile = xcd_remap(logical, n_tiles);
    const int m0 = static_cast<int>(tile / n_tiles_n) * BM;
    const int n0 = static_cast<int>(tile % n_tiles_n) * BN;
    *m0_out = m0;
    *n0_out = n0;
#pragma unroll
    for (int i = 0; i < A_PASSES; ++i) {
      const int m = m0 + a_r0 + 32 * i;
      unsigned inval = 0xFFFFFFFFu;
      int off = 0;
      if (plain_rows) {
        if (m < g.m_total) {
          inval = 0;
          off = m * g.src_ch + 4 * a_cc;
        }
      } else if (m < g.m_total) {
        const int px = m % g.p_cols;
        const int t = m / g.p_cols;
        const int py = t % g.p_rows;
        const int n = t / g.p_rows;
        const int iy0 = py * g.step_rows + g.off_rows;
        const int ix0 = px * g.step_cols + g.off_cols;
        off = ((n * g.src_rows + iy0) * g.src_cols + ix0) * g.src_ch + 4 * a_cc;
        // bit c of col_bad: tap column c falls outside the source row
        unsigned col_bad = 0;
        for (int c = 0; c < g.win_cols; ++c) {
          const unsigned ix = static_cast<unsigned>(ix0 + g.tap_sign * c);
          col_bad |= (ix < static_cast<unsigned>(g.src_cols) ? 0u : 1u) << c;
        }
        const unsigned all_cols = (1u << g.win_cols) - 1u;  // win_cols <= 31
        inval = 0;
        int shift = 0;
        for (int r = 0; r < g.win_rows; ++r, shift += g.win_cols) {
          const unsigned iy = static_cast<unsigned>(iy0 + g.tap_sign * r);
          const unsigned row =
              iy < static_cast<unsigned>(g.src_rows) ? col_bad : all_cols;
          inval |= row << shift;
        }
      }
      a_voff[i] = static_cast<unsigned>(off) * 4u;
      a_inval[i] = inval;
    }
    if (B_K_INNER) {
#pragma unroll
      for (int i = 0; i < B_PASSES; ++i) {
        const int col = n0 + b_row0 + B_ROWS_PER_PASS * i;
        b_voff[i] = col < g.n_total
                        ? static_cast<unsigned>(col * g.src_ch + 4 * b_vec) * 4u
                        : kOob;
      }
    } else {
      const int col = n0 + 4 * b_vec;
      b_voff[0] = col < g.n_total
                      ? static_cast<unsigned>(b_row0 * g.n_total + col) * 4u
                      : kOob;
    }
    tap = chunk_begin / chunks_per_tap;
    c0 = (chunk_begin - tap * chunks_per_tap) * kBK;
    tap_r = tap / g.win_cols;
    tap_c = tap - tap_r * g.win_cols;
    chunk = chunk_begin;
  };

  // Two register sets: the global loads of a chunk are issued two chunks
  // before its data is written to LDS, so their latency is covered by two
  // chunks of MFMA work (a wave of a 64x64 tile has only 16 MFMAs per chunk).
  float4 a_reg[2][A_PASSES];
  float4 b_reg[2][B_PASSES];

  auto load_global = [&](int set) {
    if (chunk >= chunk_end) return;  // wave-uniform
    const unsigned a_soff = static_cast<unsigned>(
        (g.tap_sign * (tap_r * g.src_cols + tap_c) * g.src_ch + c0) * 4);
#pragma unroll
    for (int i = 0; i < A_PASSES; ++i) {
      const unsigned bad = __builtin_amdgcn_ubfe(a_inval[i], tap, 1);
      const unsigned voff = (bad << 31) | (a_voff[i] + a_soff);
      a_reg[set][i] = __builtin_bit_cast(
          float4, __builtin_amdgcn_raw_buffer_load_b128(src_rsrc, voff, 0, 0));
    }
    if (B_K_INNER) {
      const unsigned soff =
          static_cast<unsigned>(tap) * b_tap_stride + static_cast<unsigned>(c0) * 4u;
#pragma unroll
      for (int i = 0; i < B_PASSES; ++i) {
        b_reg[set][i] = __builtin_bit_cast(
            float4,
            __builtin_amdgcn_raw_buffer_load_b128(wgt_rsrc, b_voff[i], soff, 0));
      }
    } else {
      const unsigned soff =
          static_cast<unsigned>(chunk * kBK * g.n_total) * 4u;
#pragma unroll
      for (int i = 0; i < B_PASSES; ++i) {
        b_reg[set][i] = __builtin_bit_cast(
            float4, __builtin_amdgcn_raw_buffer_load_b128(
                        wgt_rsrc, b_voff[0], soff + i * b_pass_stride, 0));
      }
    }
    // advance the scalar position by one chunk
    ++chunk;
    c0 += kBK;
    if (c0 == g.src_ch) {
      c0 = 0;
      ++tap;
      if (++tap_c == g.win_cols) { tap_c = 0; ++tap_r; }
    }
  };

  float* const a_store = lds + a_r0 * (kBK + kPad) + 4 * a_cc;
  float* const b_store =
      lds + A_FLOATS +
      (B_K_INNER ? b_row0 * (kBK + kPad) + 4 * b_vec
                 : b_row0 * (BN + kPad) + 4 * b_vec);
  auto store_tiles = [&](int stage, int set) {
#pragma unroll
    for (int i = 0; i < A_PASSES; ++i) {
      *reinterpret_cast<float4*>(a_store + stage * STAGE_FLOATS +
                                 32 * i * (kBK + kPad)) = a_reg[set][i];
    }
#pragma unroll
    for (int i = 0; i < B_PASSES; ++i) {
      constexpr int ROW_WORDS = B_K_INNER ? kBK + kPad : BN + kPad;
      *reinterpret_cast<float4*>(b_store + stage * STAGE_FLOATS +
                                 B_ROWS_PER_PASS * i * ROW_WORDS) =
          b_reg[set][i];
    }
  };

  float16v acc[TM][TN];
  auto compute = [&](int stage) {
    mma_chunk<TM, TN, true, B_K_INNER, BM, BN>(
        lds + stage * STAGE_FLOATS, lds + stage * STAGE_FLOATS + A_FLOATS,
        wave_m * WTM, wave_n * WTN, lane, acc);
  };

  const int col_l = lane & 31;
  const int row_l = 4 * (lane >> 5);
  const unsigned row_bytes = static_cast<unsigned>(g.n_total) * 4u;

  unsigned logical = blockIdx.x;
  int m0, n0;
  setup_tile(logical, &m0, &n0);
  load_global(0);  // chunk 0 of the first tile
  while (true) {
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

    // Chunk j is loaded into register set j % 2 and staged in LDS stage
    // j % 2.  The loop is unrolled by two so that stage and set are literals
    // (every LDS address is then a per-lane constant plus an immediate).
    store_tiles(0, 0);
    __syncthreads();
    load_global(1);  // chunk 1
    for (int done = 0;; done += 2) {
      load_global(0);  // chunk done + 2
      compute(0);      // chunk done
      if (done + 1 >= n_chunks) break;
      store_tiles(1, 1);  // chunk done + 1
      __syncthreads();
      load_global(1);  // chunk done + 3
      compute(1);      // chunk done + 1
      if (done + 2 >= n_chunks) break;
      store_tiles(0, 0);  // chunk done + 2
      __syncthreads();
    }

    // The next tile's addresses and its first chunk's loads, so that they
    // are in flight during the stores below.
    const int m0_done = m0, n0_done = n0;
    logical += gridDim.x;
    const bool more = logical < n_tiles;  // uniform
    if (more) {
      setup_tile(logical, &m0, &n0);
      load_global(0);
    }

    // ---- epilogue through a buffer descriptor: rows past the end fall
    // outside it and are dropped; per-lane constant offset + scalar row
    // offsets.
#pragma unroll
    for (int i = 0; i < TM; ++i) {
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const int col = n0_done + wave_n * WTN + 32 * j + col_l;
        const int m_base = m0_done + wave_m * WTM + 32 * i + row_l;
        const unsigned voff =
            (col < g.n_total && m_base < g.m_total)
                ? static_cast<unsigned>(m_base) * row_bytes +
                      static_cast<unsigned>(col) * 4u
                : kOob;
        float bias_col = 0.f;
        if (EPI) {
          if (bias != nullptr && col < g.n_total) bias_col = bias[col];
        }
        // The row offset goes into the vector offset, not the scalar offset
        // operand: hipcc (ROCm 7.2) treats buffer stores that differ only in
        // their scalar offset as stores to one address and forwards the first
        // value to all of them.
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const unsigned off =
              voff + static_cast<unsigned>(8 * (v >> 2) + (v & 3)) * row_bytes;
          float val = acc[i][j][v];
          if (EPI) {
            val += bias_col;
            if (relu) val = fmaxf(val, 0.f);
          }
          if (ATOMIC) {
            __builtin_amdgcn_raw_ptr_buffer_atomic_fadd_f32(val, dst_rsrc, off,
                                                            0, 0);
          } else {
            __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(val),
                                                  dst_rsrc, off, 0, 0);
          }
        }
      }
    }
    if (!more) break;
    // every wave is done reading the last LDS stage of this tile before the
    // next tile's first chunk is written
    __syncthreads();
  }
}

// ---------------------------------------------------------------------------
// Plain rows: C[m][n] = sum_k A[m][k] * B[k][n] with A read row by row -- the
// 1x1 stride-1 unpadded convolution (m = pixel, k = channel, n = feature) and
// the row-major matmul.  The general kernels above spend one LDS fetch
// instruction per matrix instruction on these shapes (the B operand, n
// contiguous, is fetched word by word) and store the result one word per
// lane; this kernel is built around 16-byte accesses on both sides:
//
//   * v_mfma_f32_16x16x4_f32: lane l supplies A[row l % 16][k = l / 16] and
//     B[k = l / 16][column l % 16], the 16 x 16 result sits in four registers
//     (row 4 (l / 16) + v, column l % 16);
//   * A tile [64][32 + 4], k contiguous: one ds_read_b128 gives a lane the
//     four k = 16 s + 4 (l / 16) + t, t = 0 .. 3, of its row;
//   * B tile [32][128 + 4], n contiguous: for each of those k one ds_read_b128
//     gives the lane B[k][4 (l % 16) .. + 3], which feeds FOUR matrix
//     instructions whose column blocks interleave: instruction u computes the
//     columns 4 i + u.  A lane therefore ends with four consecutive columns
//     of each of its rows and stores them with one 16-byte store;
//   * a wave owns 32 rows x 64 columns (2 x 4 blocks, 32 accumulators): per 16
//     reduction steps 6 LDS fetches feed 32 matrix instructions;
//   * a work-group is 2 x 2 waves on a 64 x 128 tile, 51 KiB of LDS in two
//     stages (three work-groups per CU).
//
//   * BM = 112 is the second tiling: 7 blocks of 16 rows, the four waves side
//     by side on 32 columns each (8-byte B fetches feeding two interleaved
//     column blocks, 56 accumulators, 8-byte stores).  The ResNet layers have
//     49 * 2^k rows; 112-row tiles divide them into counts that spread evenly
//     over the 256 CUs where 64-row tiles leave a quarter of the CUs one tile
//     more than the rest (784 tiles: 3.06 per CU).
//
// Needs k % 32 == 0, n % 4 == 0 and 16-byte aligned operands.  EPI as above.
constexpr int kRowsBN = 128;

typedef float float4v __attribute__((ext_vector_type(4)));

template <int U>
struct RowVec;
template <>
struct RowVec<4> {
  using type = float4;
  __device__ static float get(const float4& v, int u) { return comp(v, u); }
};
template <>
struct RowVec<2> {
  using type = float2;
  __device__ static float get(const float2& v, int u) {
    return u == 0 ? v.x : v.y;
  }
};

// RK: reduction steps per LDS stage, 32 or 16 (half the LDS, more work-groups
// per CU, twice the barriers).  BM: 64 (2 x 2 waves of 32 x 64) or 112 (1 x 4
// waves of 112 x 32).
template <bool EPI, int RK, int BM>
__global__ void __launch_bounds__(kThreads)
    gemm_rows_kernel(const float* __restrict__ a_ptr,
                     const float* __restrict__ b_ptr, float* __restrict__ c_ptr,
                     int m_total, int k_total, int n_total, int z_a, int z_b,
                     int z_c, unsigned n_tiles_n, unsigned n_tiles,
                     const float* __restrict__ bias, int relu) {
  static_assert(BM == 64 || BM == 112, "tilings built: 64 and 112 rows");
  constexpr int WN = BM == 64 ? 2 : 4;       // waves along n
  constexpr int RB = BM == 64 ? 2 : 7;       // 16-row blocks per wave
  constexpr int U = kRowsBN / WN / 16;       // interleaved column blocks: 4 / 2
  constexpr int A_LDS_ROWS = BM == 64 ? 64 : 128;  // copy passes of 32+ rows
  constexpr int kRowsAFloats = A_LDS_ROWS * (RK + kPad);
  constexpr int kRowsBFloats = RK * (kRowsBN + kPad);
  constexpr int kRowsStage = kRowsAFloats + kRowsBFloats;
  constexpr int A_VEC = RK / 4;                 // 16-byte pieces per A row
  constexpr int A_ROWS = kThreads / A_VEC;      // A rows per copy pass
  constexpr int A_PASSES = A_LDS_ROWS / A_ROWS;
  constexpr int B_PASSES = RK / 8;
  using BVec = typename RowVec<U>::type;
  __shared__ __align__(16) float lds[2 * kRowsStage];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave / WN, wn = wave % WN;
  const int r16 = lane & 15, g4 = lane >> 4;

  a_ptr += static_cast<size_t>(blockIdx.z) * z_a;
  b_ptr += static_cast<size_t>(blockIdx.z) * z_b;
  c_ptr += static_cast<size_t>(blockIdx.z) * z_c;
  const __amdgpu_buffer_rsrc_t a_rsrc = make_rsrc(
      a_ptr, static_cast<unsigned>(static_cast<size_t>(m_total) * k_total * 4));
  const __amdgpu_buffer_rsrc_t b_rsrc = make_rsrc(
      b_ptr, static_cast<unsigned>(static_cast<size_t>(k_total) * n_total * 4));
  const __amdgpu_buffer_rsrc_t c_rsrc = make_rsrc(
      c_ptr, static_cast<unsigned>(static_cast<size_t>(m_total) * n_total * 4));

  const unsigned tile = xcd_remap(blockIdx.x, n_tiles);
  const int m0 = static_cast<int>(tile / n_tiles_n) * BM;
  const int n0 = static_cast<int>(tile % n_tiles_n) * kRowsBN;

  // global -> register -> LDS copies: A rows tid / A_VEC + A_ROWS i, 16 bytes
  // at k quad tid % A_VEC (rows past the tile or the matrix read zeros); B
  // rows tid / 32 + 8 i, 16 bytes at column quad tid % 32
  unsigned a_off[A_PASSES], b_off[B_PASSES];
#pragma unroll
  for (int i = 0; i < A_PASSES; ++i) {
    const int row = tid / A_VEC + A_ROWS * i;
    const int m = m0 + row;
    a_off[i] = (row < BM && m < m_total)
                   ? static_cast<unsigned>(m * k_total + 4 * (tid % A_VEC)) * 4u
                   : kOob;
  }
  {
    const int col = n0 + 4 * (tid & 31);
#pragma unroll
    for (int i = 0; i < B_PASSES; ++i)
      b_off[i] = col < n_total
                     ? static_cast<unsigned>(((tid >> 5) + 8 * i) * n_total +
                                             col) * 4u
                     : kOob;
  }
  // One register set: the loads of chunk c + 1 are issued before chunk c is
  // multiplied and written to the other LDS stage after it.  (A second set,
  // loads two chunks ahead, measured 3 - 8 % slower: the extra registers cost
  // more occupancy than the longer prefetch gains.)
  float4 a_reg[A_PASSES], b_reg[B_PASSES];
  const int n_chunks = k_total / RK;
  auto load_global = [&](int chunk) {
    const unsigned a_s = static_cast<unsigned>(chunk * RK) * 4u;
    const unsigned b_s = static_cast<unsigned>(chunk * RK * n_total) * 4u;
#pragma unroll
    for (int i = 0; i < A_PASSES; ++i)
      a_reg[i] = __builtin_bit_cast(
          float4, __builtin_amdgcn_raw_buffer_load_b128(a_rsrc, a_off[i], a_s, 0));
#pragma unroll
    for (int i = 0; i < B_PASSES; ++i)
      b_reg[i] = __builtin_bit_cast(
          float4, __builtin_amdgcn_raw_buffer_load_b128(b_rsrc, b_off[i], b_s, 0));
  };
  float* const a_store =
      lds + (tid / A_VEC) * (RK + kPad) + 4 * (tid % A_VEC);
  float* const b_store =
      lds + kRowsAFloats + (tid >> 5) * (kRowsBN + kPad) + 4 * (tid & 31);
  auto store_tiles = [&](int stage) {
#pragma unroll
    for (int i = 0; i < A_PASSES; ++i)
      *reinterpret_cast<float4*>(a_store + stage * kRowsStage +
                                 A_ROWS * i * (RK + kPad)) = a_reg[i];
#pragma unroll
    for (int i = 0; i < B_PASSES; ++i)
      *reinterpret_cast<float4*>(b_store + stage * kRowsStage +
                                 8 * i * (kRowsBN + kPad)) = b_reg[i];
  };

  float4v acc[RB][U];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb)
#pragma unroll
    for (int u = 0; u < U; ++u) acc[rb][u] = float4v{0.f, 0.f, 0.f, 0.f};

  const float* const a_fetch =
      lds + (16 * RB * wm + r16) * (RK + kPad) + 4 * g4;
  const float* const b_fetch = lds + kRowsAFloats +
                               (4 * g4) * (kRowsBN + kPad) +
                               (kRowsBN / WN) * wn + U * r16;
  auto compute = [&](int stage) {
    const float* const a_tile = a_fetch + stage * kRowsStage;
    const float* const b_tile = b_fetch + stage * kRowsStage;
#pragma unroll
    for (int s = 0; s < RK / 16; ++s) {
      float4 a[RB];
      BVec b[4];
#pragma unroll
      for (int rb = 0; rb < RB; ++rb)
        a[rb] = *reinterpret_cast<const float4*>(
            a_tile + 16 * rb * (RK + kPad) + 16 * s);
#pragma unroll
      for (int t = 0; t < 4; ++t)
        b[t] = *reinterpret_cast<const BVec*>(
            b_tile + (16 * s + t) * (kRowsBN + kPad));
#pragma unroll
      for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int rb = 0; rb < RB; ++rb)
#pragma unroll
          for (int u = 0; u < U; ++u)
            acc[rb][u] = __builtin_amdgcn_mfma_f32_16x16x4f32(
                comp(a[rb], t), RowVec<U>::get(b[t], u), acc[rb][u], 0, 0, 0);
    }
  };

  load_global(0);
  store_tiles(0);
  __syncthreads();
  for (int c = 0; c < n_chunks; ++c) {
    const bool more = c + 1 < n_chunks;
    if (more) load_global(c + 1);
    compute(c & 1);
    if (more) store_tiles((c + 1) & 1);
    __syncthreads();
  }

  // lane holds C[m0 + 16 RB wm + 16 rb + 4 g4 + v][col + u], u = 0 .. U - 1
  const int col = n0 + (kRowsBN / WN) * wn + U * r16;
  float bias_u[U];
#pragma unroll
  for (int u = 0; u < U; ++u) bias_u[u] = 0.f;
  if (EPI) {
    if (bias != nullptr && col < n_total) {
#pragma unroll
      for (int u = 0; u < U; ++u) bias_u[u] = bias[col + u];
    }
  }
  const unsigned row_bytes = static_cast<unsigned>(n_total) * 4u;
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    const int row_l = 16 * RB * wm + 16 * rb + 4 * g4;  // row inside the tile
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      float out[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        out[u] = acc[rb][u][v];
        if (EPI) {
          out[u] += bias_u[u];
          if (relu) out[u] = fmaxf(out[u], 0.f);
        }
      }
      const int row = m0 + row_l + v;
      const unsigned off =
          (row_l + v < BM && row < m_total && col < n_total)
              ? static_cast<unsigned>(row) * row_bytes +
                    static_cast<unsigned>(col) * 4u
              : kOob;
      if constexpr (U == 4) {
        __builtin_amdgcn_raw_buffer_store_b128(
            __builtin_bit_cast(uint4v,
                               make_float4(out[0], out[1], out[2], out[3])),
            c_rsrc, off, 0, 2);  // written once: streaming store (slc)
      } else {
        typedef unsigned int uint2v __attribute__((ext_vector_type(2)));
        __builtin_amdgcn_raw_buffer_store_b64(
            __builtin_bit_cast(uint2v, make_float2(out[0], out[1])), c_rsrc,
            off, 0, 2);
      }
    }
  }
}

// ---------------------------------------------------------------------------
// Filter backprop: dW[q][k] = sum_m A[m][q] * dY[m][k], q = (r, s, c),
// m = (n, oy, ox).  The reduction runs over every output pixel, so both
// operands are read with the reduction index as the slow dimension and both
// LDS tiles are row-inner ([32 pixels][64 + 4]); a 64-wide q tile lies inside
// one filter tap (C % 64 == 0).  The pixel range is split across work-groups
// (blockIdx.y) and the partial tiles are added into dW with float atomics.
struct FilterBackpropGeom {
  int batch, in_rows, in_cols, channels;
  int out_rows, out_cols, features;
  int win_rows, win_cols;
  int stride_rows, stride_cols, pad_rows, pad_cols;
  int m_total;  // batch * out_rows * out_cols
};

template <typename T>
__global__ void __launch_bounds__(kThreads)
    conv_filter_backprop_kernel(const T* __restrict__ x,
                                const T* __restrict__ dy,
                                float* __restrict__ dw, FilterBackpropGeom g,
                                unsigned x_bytes, unsigned dy_bytes,
                                unsigned dw_bytes, int chunks_per_split) {
  constexpr int BM = 64, BN = 64;
  constexpr int A_FLOATS = row_inner_floats(BM);
  constexpr int STAGE_FLOATS = A_FLOATS + row_inner_floats(BN);
  __shared__ __align__(16) float lds[2 * STAGE_FLOATS];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wave_m = wave >> 1, wave_n = wave & 1;

  // tile: 64 consecutive q inside one tap x 64 features
  const int tiles_n = (g.features + BN - 1) / BN;
  const int tile_q = blockIdx.x / tiles_n;
  const int n0 = (blockIdx.x - tile_q * tiles_n) * BN;
  const int q0 = tile_q * BM;
  const int tap = q0 / g.channels;
  const int c0 = q0 - tap * g.channels;
  const int tap_r = tap / g.win_cols;
  const int tap_c = tap - tap_r * g.win_cols;

  const int n_chunks_total = (g.m_total + kBK - 1) / kBK;
  const int chunk_begin = blockIdx.y * chunks_per_split;
  const int n_chunks = min(chunks_per_split, n_chunks_total - chunk_begin);

  const __amdgpu_buffer_rsrc_t x_rsrc = make_rsrc(x, x_bytes);
  const __amdgpu_buffer_rsrc_t dy_rsrc = make_rsrc(dy, dy_bytes);

  // This lane copies float4 `vec` of pixel rows row0 and row0 + 16 of every
  // 32-pixel chunk, for both operands.
  const int vec = tid & 15;
  const int row0 = tid >> 4;
  int ox[2], iy[2];      // output column; input row of this tap
  int x_off[2];          // element offset of (n, iy, ox*stride - pad + tap_c, c0 + 4*vec)
  unsigned dy_off[2];    // byte offset of (m, n0 + 4*vec)
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int m = chunk_begin * kBK + row0 + 16 * i;
    const int o = m % g.out_cols;
    const int t = m / g.out_cols;
    const int oy = t % g.out_rows;
    const int n = t / g.out_rows;
    ox[i] = o;
    iy[i] = oy * g.stride_rows - g.pad_rows + tap_r;
    x_off[i] = ((n * g.in_rows + iy[i]) * g.in_cols + o * g.stride_cols -
                g.pad_cols + tap_c) * g.channels + c0 + 4 * vec;
    dy_off[i] = (n0 + 4 * vec < g.features)
                    ? static_cast<unsigned>(m * g.features + n0 + 4 * vec) *
                          static_cast<unsigned>(sizeof(T))
                    : kOob;
  }
  // element-offset deltas of the pixel walk
  const int step_px = g.stride_cols * g.channels;  // ox += 1
  const int step_row =
      (g.stride_rows * g.in_cols - g.out_cols * g.stride_cols) * g.channels;
  const int step_img =
      (g.in_rows - g.out_rows * g.stride_rows) * g.in_cols * g.channels;
  const int iy_first = -g.pad_rows + tap_r;
  const int iy_end = iy_first + g.out_rows * g.stride_rows;

  float4 a_reg[2], b_reg[2];
  auto load_global = [&]() {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int ix = ox[i] * g.stride_cols - g.pad_cols + tap_c;
      const bool ok =
          (static_cast<unsigned>(iy[i]) < static_cast<unsigned>(g.in_rows)) &
          (static_cast<unsigned>(ix) < static_cast<unsigned>(g.in_cols));
      a_reg[i] = buffer_load4_as_float<T>(
          x_rsrc, ok ? static_cast<unsigned>(x_off[i]) *
                           static_cast<unsigned>(sizeof(T))
                     : kOob);
      b_reg[i] = buffer_load4_as_float<T>(dy_rsrc, dy_off[i]);
      // advance this row by one chunk (32 pixels)
      ox[i] += kBK;
      x_off[i] += kBK * step_px;
      while (ox[i] >= g.out_cols) {
        ox[i] -= g.out_cols;
        x_off[i] += step_row;
        iy[i] += g.stride_rows;
        if (iy[i] == iy_end) {
          iy[i] = iy_first;
          x_off[i] += step_img;
        }
      }
      if (dy_off[i] != kOob)
        dy_off[i] += kBK * g.features * static_cast<unsigned>(sizeof(T));
    }
  };
  float* const a_store = lds + row0 * (BM + kPad) + 4 * vec;
  float* const b_store = lds + A_FLOATS + row0 * (BN + kPad) + 4 * vec;
  auto store_tiles = [&](int stage) {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      *reinterpret_cast<float4*>(a_store + stage * STAGE_FLOATS +
                                 16 * i * (BM + kPad)) = a_reg[i];
      *reinterpret_cast<float4*>(b_store + stage * STAGE_FLOATS +
                                 16 * i * (BN + kPad)) = b_reg[i];
    }
  };

  float16v acc[1][1];
#pragma unroll
  for (int v = 0; v < 16; ++v) acc[0][0][v] = 0.f;
  auto compute = [&](int stage) {
    mma_chunk<1, 1, false, false, BM, BN>(
        lds + stage * STAGE_FLOATS, lds + stage * STAGE_FLOATS + A_FLOATS,
        wave_m * 32, wave_n * 32, lane, acc);
  };

  load_global();
  store_tiles(0);
  __syncthreads();
  for (int done = 0;; done += 2) {
    if (done + 1 < n_chunks) load_global();
    compute(0);
    if (done + 1 >= n_chunks) break;
    store_tiles(1);
    __syncthreads();
    if (done + 2 < n_chunks) load_global();
    compute(1);
    if (done + 2 >= n_chunks) break;
    store_tiles(0);
    __syncthreads();
  }

  const __amdgpu_buffer_rsrc_t dw_rsrc = make_rsrc(dw, dw_bytes);
  const int col = n0 + wave_n * 32 + (lane & 31);
  const int q_base = q0 + wave_m * 32 + 4 * (lane >> 5);
  const unsigned row_bytes = static_cast<unsigned>(g.features) * 4u;
  const unsigned voff = col < g.features
                            ? static_cast<unsigned>(q_base) * row_bytes +
                                  static_cast<unsigned>(col) * 4u
                            : kOob;
#pragma unroll
  for (int v = 0; v < 16; ++v) {
    const unsigned off =
        voff + static_cast<unsigned>(8 * (v >> 2) + (v & 3)) * row_bytes;
    const float val = acc[0][0][v];
    __builtin_amdgcn_raw_ptr_buffer_atomic_fadd_f32(val, dw_rsrc, off, 0, 0);
  }
}

// Filter backprop for layers with few input channels (the 7x7x3 stem): the
// whole (tap, channel) range q = 0 .. R*S*C - 1 (at most 192) fits one
// work-group, which therefore owns all of dW for 64 features and walks a
// range of output pixels, 32 per chunk.  A tile: [32 pixels][q], gathered
// element by element (consecutive q are not aligned runs of the input);
// rows are 193 floats apart so that lanes that differ in the pixel hit
// different banks.  The up to 6 x 2 accumulator blocks are dealt to the four
// waves round-robin.  Partial sums meet in dW through float atomics.
// Layers with at most eight channels and a longer (tap, channel) range (an
// 11x11x3 stem: 363) run as up to kSmallQParts parts of 192 in blockIdx.z,
// each part an independent launch of the same scheme over its rows of dW.
constexpr int kSmallQMax = 192;
constexpr int kSmallQStride = kSmallQMax + 1;
constexpr int kSmallQParts = 4;
constexpr int kSmallQPartsMaxChannels = 8;

__global__ void __launch_bounds__(kThreads)
    conv_filter_backprop_smallq_kernel(const float* __restrict__ x,
                                       const float* __restrict__ dy,
                                       float* __restrict__ dw,
                                       FilterBackpropGeom g, unsigned x_bytes,
                                       unsigned dy_bytes, unsigned dw_bytes,
                                       int chunks_per_split) {
  constexpr int BN = 64;
  constexpr int A_FLOATS = kBK * kSmallQStride;
  constexpr int STAGE_FLOATS = A_FLOATS + row_inner_floats(BN);
  extern __shared__ __align__(16) float lds[];  // 2 * STAGE_FLOATS (65.25 KiB)

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n0 = blockIdx.x * BN;
  // this part's rows of dW: q_begin .. q_begin + q_total - 1
  const int q_begin = blockIdx.z * kSmallQMax;
  const int q_total =
      min(kSmallQMax, g.win_rows * g.win_cols * g.channels - q_begin);
  const int n_mblocks = (q_total + 31) / 32;
  const int n_blocks = 2 * n_mblocks;

  const int n_chunks_total = (g.m_total + kBK - 1) / kBK;
  const int chunk_begin = blockIdx.y * chunks_per_split;
  const int n_chunks = min(chunks_per_split, n_chunks_total - chunk_begin);

  const __amdgpu_buffer_rsrc_t x_rsrc = make_rsrc(x, x_bytes);
  const __amdgpu_buffer_rsrc_t dy_rsrc = make_rsrc(dy, dy_bytes);

  // A gather: this lane owns pixel `a_px` of every chunk and the 24
  // consecutive q starting at a_q0.
  constexpr int A_PER_LANE = kSmallQMax * kBK / kThreads;  // 24
  const int a_px = tid & 31;
  const int a_q0 = (tid >> 5) * A_PER_LANE;
  int a_ox, a_iy0, a_base;  // output column, first input row, element offset
  {
    const int m = chunk_begin * kBK + a_px;
    a_ox = m % g.out_cols;
    const int t = m / g.out_cols;
    const int oy = t % g.out_rows;
    const int n = t / g.out_rows;
    a_iy0 = oy * g.stride_rows - g.pad_rows;
    a_base = ((n * g.in_rows + a_iy0) * g.in_cols + a_ox * g.stride_cols -
              g.pad_cols) * g.channels;
  }
  const int step_px = g.stride_cols * g.channels;
  const int step_row =
      (g.stride_rows * g.in_cols - g.out_cols * g.stride_cols) * g.channels;
  const int step_img =
      (g.in_rows - g.out_rows * g.stride_rows) * g.in_cols * g.channels;
  const int iy_end = -g.pad_rows + g.out_rows * g.stride_rows;
  // (tap row, tap col, channel) of a_q0
  int q_r, q_s, q_c;
  {
    const int tap = (q_begin + a_q0) / g.channels;
    q_c = q_begin + a_q0 - tap * g.channels;
    q_r = tap / g.win_cols;
    q_s = tap - q_r * g.win_cols;
  }
  // B copy: float4 `b_vec` of pixel rows b_row0 and b_row0 + 16
  const int b_vec = tid & 15;
  const int b_row0 = tid >> 4;
  unsigned dy_off[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int m = chunk_begin * kBK + b_row0 + 16 * i;
    dy_off[i] = (n0 + 4 * b_vec < g.features)
                    ? static_cast<unsigned>(m * g.features + n0 + 4 * b_vec) * 4u
                    : kOob;
  }

  float a_reg[A_PER_LANE];
  float4 b_reg[2];
  auto load_global = [&]() {
    const int ix0 = a_ox * g.stride_cols - g.pad_cols;
    int r = q_r, sc = q_s, c = q_c;
#pragma unroll
    for (int j = 0; j < A_PER_LANE; ++j) {
      const int iy = a_iy0 + r;
      const int ix = ix0 + sc;
      const bool ok =
          (a_q0 + j < q_total) &
          (static_cast<unsigned>(iy) < static_cast<unsigned>(g.in_rows)) &
          (static_cast<unsigned>(ix) < static_cast<unsigned>(g.in_cols));
      const int off = a_base + (r * g.in_cols + sc) * g.channels + c;
      a_reg[j] = __builtin_bit_cast(
          float, __builtin_amdgcn_raw_buffer_load_b32(
                     x_rsrc, ok ? static_cast<unsigned>(off) * 4u : kOob, 0,
                     0));
      if (++c == g.channels) {
        c = 0;
        if (++sc == g.win_cols) { sc = 0; ++r; }
      }
    }
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      b_reg[i] = buffer_load4(dy_rsrc, dy_off[i]);
      if (dy_off[i] != kOob) dy_off[i] += kBK * g.features * 4u;
    }
    // advance the pixel by one chunk
    a_ox += kBK;
    a_base += kBK * step_px;
    while (a_ox >= g.out_cols) {
      a_ox -= g.out_cols;
      a_base += step_row;
      a_iy0 += g.stride_rows;
      if (a_iy0 == iy_end) {
        a_iy0 = -g.pad_rows;
        a_base += step_img;
      }
    }
  };
  float* const a_store = lds + a_px * kSmallQStride + a_q0;
  float* const b_store = lds + A_FLOATS + b_row0 * (BN + kPad) + 4 * b_vec;
  auto store_tiles = [&](int stage) {
#pragma unroll
    for (int j = 0; j < A_PER_LANE; ++j)
      a_store[stage * STAGE_FLOATS + j] = a_reg[j];
#pragma unroll
    for (int i = 0; i < 2; ++i)
      *reinterpret_cast<float4*>(b_store + stage * STAGE_FLOATS +
                                 16 * i * (BN + kPad)) = b_reg[i];
  };

  constexpr int BLOCKS_PER_WAVE = 3;  // 12 blocks over 4 waves
  float16v acc[BLOCKS_PER_WAVE];
#pragma unroll
  for (int i = 0; i < BLOCKS_PER_WAVE; ++i)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[i][v] = 0.f;
  const int l32 = lane & 31;
  auto compute = [&](int stage) {
    const float* a_tile = lds + stage * STAGE_FLOATS;
    const float* b_tile = a_tile + A_FLOATS;
#pragma unroll
    for (int i = 0; i < BLOCKS_PER_WAVE; ++i) {
      const int blk = wave + 4 * i;
      if (blk >= n_blocks) break;
      const int mb = blk >> 1, nb = blk & 1;
      float4 a[kBK / 8], b[kBK / 8];
#pragma unroll
      for (int s4 = 0; s4 < kBK / 8; ++s4) {
        a[s4] = fetch_row_inner<kSmallQStride - kPad>(a_tile, mb * 32 + l32,
                                                      s4, lane);
        b[s4] = fetch_row_inner<BN>(b_tile, nb * 32 + l32, s4, lane);
      }
#pragma unroll
      for (int s4 = 0; s4 < kBK / 8; ++s4)
#pragma unroll
        for (int t = 0; t < 4; ++t)
          acc[i] = __builtin_amdgcn_mfma_f32_32x32x2f32(
              comp(a[s4], t), comp(b[s4], t), acc[i], 0, 0, 0);
    }
  };

  load_global();
  store_tiles(0);
  __syncthreads();
  for (int done = 0; done < n_chunks; ++done) {
    const int stage = done & 1;
    const bool more = done + 1 < n_chunks;
    if (more) load_global();
    compute(stage);
    if (more) store_tiles(stage ^ 1);
    __syncthreads();
  }

  const __amdgpu_buffer_rsrc_t dw_rsrc = make_rsrc(dw, dw_bytes);
  const unsigned row_bytes = static_cast<unsigned>(g.features) * 4u;
#pragma unroll
  for (int i = 0; i < BLOCKS_PER_WAVE; ++i) {
    const int blk = wave + 4 * i;
    if (blk >= n_blocks) break;
    const int mb = blk >> 1, nb = blk & 1;
    const int col = n0 + nb * 32 + l32;
    const int q_base = mb * 32 + 4 * (lane >> 5);
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int q = q_base + 8 * (v >> 2) + (v & 3);
      const unsigned off =
          (col < g.features && q < q_total)
              ? static_cast<unsigned>(q_begin + q) * row_bytes +
                    static_cast<unsigned>(col) * 4u
              : kOob;
      __builtin_amdgcn_raw_ptr_buffer_atomic_fadd_f32(acc[i][v], dw_rsrc, off,
                                                      0, 0);
    }
  }
}

// Second half of the input gradient for layers with very few input channels
// (the stem): Z[m][(r, s, c)] = sum_k dY[m][k] * W[r][s][c][k] has been
// computed as one GEMM over the output pixels m; every input element then
// sums the Z entries of the taps that reach it,
//   dX[n][y][x][c] = sum_{r,s} Z[(n, (y+pad-r)/stride, (x+pad-s)/stride)][r][s][c]
// over the taps for which the divisions are exact and in range.  One lane per
// dX element, channel fastest.
__global__ void __launch_bounds__(256)
    col2im_gather_kernel(const float* __restrict__ z, float* __restrict__ dx,
                         FilterBackpropGeom g, int images) {
  const size_t idx = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
  const size_t total =
      static_cast<size_t>(images) * g.in_rows * g.in_cols * g.channels;
  if (idx >= total) return;
  const int c = static_cast<int>(idx % g.channels);
  size_t t = idx / g.channels;
  const int xx = static_cast<int>(t % g.in_cols);
  t /= g.in_cols;
  const int yy = static_cast<int>(t % g.in_rows);
  const int n = static_cast<int>(t / g.in_rows);
  const int q_total = g.win_rows * g.win_cols * g.channels;
  float acc = 0.f;
  for (int r = 0; r < g.win_rows; ++r) {
    const int ty = yy + g.pad_rows - r;
    if (ty < 0 || ty % g.stride_rows != 0) continue;
    const int oy = ty / g.stride_rows;
    if (oy >= g.out_rows) continue;
    for (int sc = 0; sc < g.win_cols; ++sc) {
      const int tx = xx + g.pad_cols - sc;
      if (tx < 0 || tx % g.stride_cols != 0) continue;
      const int ox = tx / g.stride_cols;
      if (ox >= g.out_cols) continue;
      acc += z[(static_cast<size_t>(n * g.out_rows + oy) * g.out_cols + ox) *
                   q_total +
               (r * g.win_cols + sc) * g.channels + c];
    }
  }
  dx[idx] = acc;
}

__global__ void __launch_bounds__(256)
    zero_fill_kernel(float4* __restrict__ p, size_t n_vec) {
  const size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
  if (i < n_vec) p[i] = make_float4(0.f, 0.f, 0.f, 0.f);
}

// Number of work-groups along x for the fast kernel, which walks tiles
// x, x + gridDim.x, ...: as many as the GPU holds at once (CUs times the
// work-groups of this kernel one CU can host), shared between the `yz`
// reduction splits and batches of the launch, in whole rounds of the 8 XCDs;
// one work-group per tile when there are fewer than four tiles for each.
template <typename Kernel>
unsigned resident_groups(Kernel kernel, size_t lds_bytes) {
  int per_cu = 0, device = 0, cus = 0;
  if (hipOccupancyMaxActiveBlocksPerMultiprocessor(
          &per_cu, reinterpret_cast<const void*>(kernel), kThreads,
          lds_bytes) != hipSuccess ||
      hipGetDevice(&device) != hipSuccess ||
      hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount,
                            device) != hipSuccess) {
    (void)hipGetLastError();
    return 0;
  }
  return static_cast<unsigned>(max(per_cu, 1)) * static_cast<unsigned>(cus);
}

inline unsigned persistent_grid_x(unsigned resident, unsigned n_tiles,
                                  unsigned yz) {
  static const bool off = SNN_TUNING_ENV("SNN_HIP_IGEMM_ONE_TILE") != nullptr;
  if (off || resident == 0) return n_tiles;
  unsigned gx = resident / max(yz, 1u);
  gx -= gx % 8u;
  if (gx < 8u) gx = 8u;
  // Tiles are dealt round-robin, so with only a few per work-group the
  // uneven shares cost more than the saved dispatches (measured: 1.5 tiles
  // per work-group ran 20 % slower than one work-group per tile).
  return n_tiles >= 4u * gx ? gx : n_tiles;
}

template <int BM, int BN, int WM, int WN, bool B_K_INNER, bool STRIDED>
void launch_tile(const float* src, const float* wgt, float* dst,
                 const Gather& g, size_t src_elems, size_t wgt_elems,
                 int splits, hipStream_t stream, int batches = 1,
                 bool accumulate = false,
                 const LaunchOptions* epilogue = nullptr) {
  // accumulate: add the product to what dst holds (atomic kernel, no zero
  // fill) instead of overwriting it.
  const unsigned tiles_m = static_cast<unsigned>(ceil_div(g.m_total, BM));
  const unsigned tiles_n = static_cast<unsigned>(ceil_div(g.n_total, BN));
  const unsigned n_tiles = tiles_m * tiles_n;
  const int n_chunks = ceil_div(g.k_total, kBK);
  const int per_split = ceil_div(n_chunks, splits);
  splits = ceil_div(n_chunks, per_split);
  constexpr size_t kLdsBytes =
      2 * sizeof(float) *
      (k_inner_floats(BM) +
       (B_K_INNER ? k_inner_floats(BN) : row_inner_floats(BN)));
  const unsigned src_bytes = static_cast<unsigned>(src_elems * sizeof(float));
  const unsigned wgt_bytes = static_cast<unsigned>(wgt_elems * sizeof(float));
  const bool fast = !STRIDED && g.src_ch % kBK == 0 &&
                    g.win_rows * g.win_cols <= 32;
  const unsigned dst_bytes = static_cast<unsigned>(
      static_cast<size_t>(g.m_total) * g.n_total * sizeof(float));
  if (splits > 1 || accumulate) {
    // Partial sums meet in the output through float atomics: start from zero.
    // (a batched launch keeps its problems contiguous: z_dst == m * n)
    const size_t n_vec = static_cast<size_t>(batches) * g.m_total *
                         g.n_total / 4;  // a multiple of 4 elements
    if (!accumulate)
      hipLaunchKernelGGL(
          zero_fill_kernel,
          dim3(static_cast<unsigned>(ceil_div(n_vec, size_t{256}))), dim3(256),
          0, stream, reinterpret_cast<float4*>(dst), n_vec);
    KernelTimer timer(stream);
    if (fast) {
      auto kernel = conv_igemm_fast_kernel<BM, BN, WM, WN, B_K_INNER, true>;
      static const hipError_t attr = hipFuncSetAttribute(
          reinterpret_cast<const void*>(kernel),
          hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes);
      (void)attr;
      static const unsigned resident = resident_groups(kernel, kLdsBytes);
      const unsigned gx = persistent_grid_x(
          resident, n_tiles, static_cast<unsigned>(splits * batches));
      hipLaunchKernelGGL(kernel, dim3(gx, splits, batches),
                         dim3(kThreads), kLdsBytes, stream, src, wgt, dst, g,
                         src_bytes, wgt_bytes, dst_bytes, tiles_n, n_tiles,
                         per_split, static_cast<const float*>(nullptr), 0);
      return;
    }
    auto kernel = conv_igemm_kernel<BM, BN, WM, WN, B_K_INNER, STRIDED, true>;
    static const hipError_t attr = hipFuncSetAttribute(
        reinterpret_cast<const void*>(kernel),
        hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes);
    (void)attr;
    hipLaunchKernelGGL(kernel, dim3(n_tiles, splits), dim3(kThreads),
                       kLdsBytes, stream, src, wgt, dst, g, src_bytes,
                       wgt_bytes, tiles_n, n_tiles, per_split);
  } else {
    KernelTimer timer(stream);
    if (fast && epilogue != nullptr && epilogue->wanted() && batches == 1) {
      auto kernel =
          conv_igemm_fast_kernel<BM, BN, WM, WN, B_K_INNER, false, true>;
      static const hipError_t attr = hipFuncSetAttribute(
          reinterpret_cast<const void*>(kernel),
          hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes);
      (void)attr;
      static const unsigned resident = resident_groups(kernel, kLdsBytes);
      const unsigned gx = persistent_grid_x(resident, n_tiles, 1u);
      hipLaunchKernelGGL(kernel, dim3(gx, 1, 1), dim3(kThreads),
                         kLdsBytes, stream, src, wgt, dst, g, src_bytes,
                         wgt_bytes, dst_bytes, tiles_n, n_tiles, per_split,
                         epilogue->bias, epilogue->relu ? 1 : 0);
      if (epilogue->applied != nullptr) *epilogue->applied = true;
      return;
    }
    if (fast) {
      auto kernel = conv_igemm_fast_kernel<BM, BN, WM, WN, B_K_INNER, false>;
      static const hipError_t attr = hipFuncSetAttribute(
          reinterpret_cast<const void*>(kernel),
          hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes);
      (void)attr;
      static const unsigned resident = resident_groups(kernel, kLdsBytes);
      const unsigned gx = persistent_grid_x(
          resident, n_tiles, static_cast<unsigned>(batches));
      hipLaunchKernelGGL(kernel, dim3(gx, 1, batches), dim3(kThreads),
                         kLdsBytes, stream, src, wgt, dst, g, src_bytes,
                         wgt_bytes, dst_bytes, tiles_n, n_tiles, per_split,
                         static_cast<const float*>(nullptr), 0);
      return;
    }
    auto kernel = conv_igemm_kernel<BM, BN, WM, WN, B_K_INNER, STRIDED, false>;
    // More than the 64 KiB default needs an explicit opt-in (160 KiB per CU).
    static const hipError_t attr = hipFuncSetAttribute(
        reinterpret_cast<const void*>(kernel),
        hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes);
    (void)attr;
    hipLaunchKernelGGL(kernel, dim3(n_tiles, 1), dim3(kThreads), kLdsBytes,
                       stream, src, wgt, dst, g, src_bytes, wgt_bytes, tiles_n,
                       n_tiles, per_split);
  }
}

// Tile shape and reduction split.  Measured on MI355X with the ResNet layers:
// 64x64 tiles (four work-groups resident per CU) beat the larger tiles unless
// the problem is several times bigger than the chip, because a launch only
// lasts a few dozen chunk times and balance across the 256 CUs matters more
// than per-tile reuse.  When 64x64 tiles number fewer than one per resident
// slot, the reduction is split across work-groups so that there are about
// kSplitUnits work units; their partial sums meet in the output through float
// atomics (the order of those additions is not fixed, so the last bits of
// such outputs can differ from run to run).
constexpr int kResidentSlots = 1024;  // 256 CUs x 4 work-groups of 64x64
constexpr int kSplitUnits = 2048;
constexpr int kMinChunksPerSplit = 8;

// The plain-rows kernel: one work-group per BM x 128 tile, `batches`
// independent problems along blockIdx.z.
//  * BM: the work-groups spread over the 256 CUs, so a launch lasts about
//    ceil(tiles / 256) * BM row-steps; 112-row tiles are taken when that is
//    smaller than for 64-row tiles (49 * 2^k rows: 3.06 tiles per CU become
//    1.75).
//  * RK: stages of 32 reduction steps or of 16 (more work-groups resident per
//    CU at twice the barriers); the shorter stage when it saves a round of
//    work-groups.
template <bool EPI, int RK, int BM>
void launch_gemm_rows_as(const float* a, const float* b, float* c, int m,
                         int k, int n, int batches, int z_a, int z_b, int z_c,
                         const float* bias, int relu, hipStream_t stream) {
  const unsigned tiles_m = static_cast<unsigned>(ceil_div(m, BM));
  const unsigned tiles_n = static_cast<unsigned>(ceil_div(n, kRowsBN));
  const unsigned n_tiles = tiles_m * tiles_n;
  hipLaunchKernelGGL((gemm_rows_kernel<EPI, RK, BM>),
                     dim3(n_tiles, 1, static_cast<unsigned>(batches)),
                     dim3(kThreads), 0, stream, a, b, c, m, k, n, z_a, z_b, z_c,
                     tiles_n, n_tiles, bias, relu);
}

void launch_gemm_rows(const float* a, const float* b, float* c, int m, int k,
                      int n, int batches, int z_a, int z_b, int z_c,
                      hipStream_t stream, const LaunchOptions* epilogue) {
  const long tiles_n = ceil_div(n, kRowsBN);
  const long groups64 = static_cast<long>(ceil_div(m, 64)) * tiles_n * batches;
  const long groups112 =
      static_cast<long>(ceil_div(m, 112)) * tiles_n * batches;
  // (measured: a 6 % shorter estimate -- 56x56x64 -> 256 -- changes nothing,
  // and 224 work-groups of four waves cannot fill 256 CUs -- 7x7x512 -> 2048 --
  // so the tall tile needs a tenth less and at least 320 work-groups)
  bool tall = 10 * ((groups112 + 255) / 256) * 112 <=
                  9 * ((groups64 + 255) / 256) * 64 &&
              groups112 >= 320;
  if (const char* tune = SNN_TUNING_ENV("SNN_HIP_GEMM_ROWS_BM")) {
    if (tune[0] != 0) tall = std::atoi(tune) == 112;
  }
  const long groups = tall ? groups112 : groups64;
  // resident work-groups on 256 CUs: 64-row tiles 3 / 5 per CU (stage of 32 /
  // 16 steps), 112-row tiles 2 / 4
  const long slots32 = tall ? 512 : 768, slots16 = tall ? 1024 : 1280;
  bool short_stage =
      (groups + slots16 - 1) / slots16 < (groups + slots32 - 1) / slots32;
  if (const char* tune = SNN_TUNING_ENV("SNN_HIP_GEMM_ROWS_RK")) {
    if (tune[0] != 0) short_stage = std::atoi(tune) == 16;
  }
  KernelTimer timer(stream);
  // bias is added per column from the bias vector
  const bool fuse = epilogue != nullptr && epilogue->wanted() && batches == 1;
  const float* bias = fuse ? epilogue->bias : nullptr;
  const int relu = fuse && epilogue->relu ? 1 : 0;
  // short reductions: the kernel that keeps the filter in registers
  if (batches == 1 && gemm_wreg_supports(m, k, n) &&
      SNN_TUNING_ENV("SNN_HIP_GEMM_WREG_OFF") == nullptr) {
    launch_gemm_wreg(a, b, c, m, k, n, fuse, bias, relu != 0, stream);
    if (fuse && epilogue->applied != nullptr) *epilogue->applied = true;
    return;
  }
#define SNN_ROWS(EPI, RK, BM)                                                 \
  launch_gemm_rows_as<EPI, RK, BM>(a, b, c, m, k, n, batches, z_a, z_b, z_c, \
                                   bias, relu, stream)
  if (fuse) {
    if (tall) {
      if (short_stage) SNN_ROWS(true, 16, 112); else SNN_ROWS(true, 32, 112);
    } else {
      if (short_stage) SNN_ROWS(true, 16, 64); else SNN_ROWS(true, 32, 64);
    }
    if (epilogue->applied != nullptr) *epilogue->applied = true;
  } else {
    if (tall) {
      if (short_stage) SNN_ROWS(false, 16, 112); else SNN_ROWS(false, 32, 112);
    } else {
      if (short_stage) SNN_ROWS(false, 16, 64); else SNN_ROWS(false, 32, 64);
    }
  }
#undef SNN_ROWS
}

// Shapes the plain-rows kernel takes and is the better choice for: rows read
// as they are, k in whole chunks, 16-byte columns, and enough 64 x 128 tiles
// to give every CU a work-group (smaller problems keep the 64 x 64 tiles and
// the reduction split of the general kernel).  (The same kernel with the
// im2col gather of conv_igemm_fast_kernel in front was measured on the 3x3
// ResNet layers: within 3 % of that kernel either way, so convolutions with a
// window keep the general kernel.)
constexpr long kRowsMinTiles = 256;
bool gemm_rows_wanted(int m, int k, int n, int batches) {
  static const char* tune = SNN_TUNING_ENV("SNN_HIP_GEMM_ROWS");
  if (tune != nullptr && tune[0] == '0') return false;
  const long tiles = static_cast<long>(ceil_div(m, 64)) *
                     ceil_div(n, kRowsBN) * batches;
  const long min_tiles = (tune != nullptr && tune[0] == '1') ? 1 : kRowsMinTiles;
  // columns past n in the last 128-wide tile are computed and dropped: at
  // most a fifth of the work
  const int n_padded = ceil_div(n, kRowsBN) * kRowsBN;
  return k % kBK == 0 && n % 4 == 0 && tiles >= min_tiles &&
         5 * (n_padded - n) <= n_padded;
}

template <bool B_K_INNER, bool STRIDED>
void launch_auto(const float* src, const float* wgt, float* dst,
                 const Gather& g, size_t src_elems, size_t wgt_elems,
                 hipStream_t stream, const LaunchOptions* epilogue = nullptr) {
  auto tiles = [&](int bm, int bn) {
    return static_cast<long>(ceil_div(g.m_total, bm)) * ceil_div(g.n_total, bn);
  };
  const int n_chunks = ceil_div(g.k_total, kBK);
  if constexpr (!B_K_INNER && !STRIDED) {
    const bool plain_rows = g.win_rows == 1 && g.win_cols == 1 &&
                            g.step_rows == 1 && g.step_cols == 1 &&
                            g.off_rows == 0 && g.off_cols == 0 &&
                            g.src_rows == g.p_rows && g.src_cols == g.p_cols;
    // (64-feature filters are too narrow for the plain-rows tiles, not for
    // the filter-in-registers kernel it hands short reductions to)
    if (plain_rows &&
        (gemm_rows_wanted(g.m_total, g.k_total, g.n_total, 1) ||
         (gemm_wreg_supports(g.m_total, g.k_total, g.n_total) &&
          SNN_TUNING_ENV("SNN_HIP_GEMM_WREG_OFF") == nullptr))) {
      launch_gemm_rows(src, wgt, dst, g.m_total, g.k_total, g.n_total, 1, 0, 0,
                       0, stream, epilogue);
      return;
    }
  }
  if constexpr (B_K_INNER && !STRIDED) {
    // The input gradient of a 1x1 stride-1 unpadded convolution is the plain
    // product dX[m][c] = sum_k dY[m][k] W[c][k]: with few enough features
    // (the reduction) the kernel that keeps the filter in registers takes it,
    // reading W as it is stored.
    const bool plain_rows = g.win_rows == 1 && g.win_cols == 1 &&
                            g.step_rows == 1 && g.step_cols == 1 &&
                            g.off_rows == 0 && g.off_cols == 0 &&
                            g.src_rows == g.p_rows && g.src_cols == g.p_cols &&
                            g.div_rows == 1 && g.div_cols == 1;
    if (plain_rows &&
        gemm_wreg_supports(g.m_total, g.k_total, g.n_total, true) &&
        SNN_TUNING_ENV("SNN_HIP_GEMM_WREG_OFF") == nullptr) {
      KernelTimer timer(stream);
      launch_gemm_wreg(src, wgt, dst, g.m_total, g.k_total, g.n_total, false,
                       nullptr, false, stream, true);
      return;
    }
  }
  // Developer override for tuning runs: SNN_HIP_IGEMM="<tile>,<splits>" with
  // tile 0 = 128x128, 1 = 128x64, 2 = 64x64.
  static const char* tune = SNN_TUNING_ENV("SNN_HIP_IGEMM");
  if (tune != nullptr) {
    int tile = 2, splits = 1;
    sscanf(tune, "%d,%d", &tile, &splits);
    splits = max(1, min(splits, n_chunks));
    if (g.n_total % 4 != 0) splits = 1;
    if (tile == 0)
      launch_tile<128, 128, 2, 2, B_K_INNER, STRIDED>(
          src, wgt, dst, g, src_elems, wgt_elems, splits, stream);
    else if (tile == 1)
      launch_tile<128, 64, 4, 1, B_K_INNER, STRIDED>(
          src, wgt, dst, g, src_elems, wgt_elems, splits, stream);

    else
      launch_tile<64, 64, 2, 2, B_K_INNER, STRIDED>(
          src, wgt, dst, g, src_elems, wgt_elems, splits, stream);
    return;
  }
  if (g.n_total > 64 && tiles(128, 128) >= 4 * kResidentSlots) {
    launch_tile<128, 128, 2, 2, B_K_INNER, STRIDED>(
        src, wgt, dst, g, src_elems, wgt_elems, 1, stream, 1, false, epilogue);
    return;
  }
  const long t = tiles(64, 64);
  int splits = 1;
  // n_total % 4 == 0 is needed by the zero fill of the split path
  // (measured: 800 tiles run 5 % faster unsplit than in two halves plus the
  // zero fill, so a launch that nearly fills the slots is left alone)
  const bool deterministic = epilogue != nullptr && epilogue->deterministic;
  if (t < kResidentSlots * 5 / 8 && g.n_total % 4 == 0 && !deterministic) {
    splits = static_cast<int>((kSplitUnits + t - 1) / t);
    splits = max(1, min(splits, n_chunks / kMinChunksPerSplit));
  }
  launch_tile<64, 64, 2, 2, B_K_INNER, STRIDED>(
      src, wgt, dst, g, src_elems, wgt_elems, splits, stream, 1, false,
      epilogue);
}

// Forward convolution whose channel count is not a multiple of 4: 64x64
// tiles, scalar gather, no reduction split (such layers have few channels
// and many pixels).
void launch_scalar_gather_forward(const float* src, const float* wgt,
                                  float* dst, const Gather& g,
                                  size_t src_elems, size_t wgt_elems,
                                  hipStream_t stream) {
  constexpr int BM = 64, BN = 64;
  const unsigned tiles_m = static_cast<unsigned>(ceil_div(g.m_total, BM));
  const unsigned tiles_n = static_cast<unsigned>(ceil_div(g.n_total, BN));
  const unsigned n_tiles = tiles_m * tiles_n;
  const int n_chunks = ceil_div(g.k_total, kBK);
  constexpr size_t kLdsBytes =
      2 * sizeof(float) * (k_inner_floats(BM) + row_inner_floats(BN));
  auto kernel = conv_igemm_kernel<BM, BN, 2, 2, false, false, false, true>;
  static const hipError_t attr = hipFuncSetAttribute(
      reinterpret_cast<const void*>(kernel),
      hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes);
  (void)attr;
  KernelTimer timer(stream);
  hipLaunchKernelGGL(kernel, dim3(n_tiles, 1), dim3(kThreads), kLdsBytes,
                     stream, src, wgt, dst, g,
                     static_cast<unsigned>(src_elems * sizeof(float)),
                     static_cast<unsigned>(wgt_elems * sizeof(float)), tiles_n,
                     n_tiles, n_chunks);
}

}  // namespace

// Input gradient with very few input channels: as a GEMM over (r, s, k) the
// 3 output columns would waste 29/32 of every matrix instruction, so the
// product is taken per output pixel against all (r, s, c) at once (a 1x1
// "convolution" of dY with R*S*C features, the HWCF filter being exactly the
// K-contiguous operand that needs) and col2im_gather_kernel folds the taps.
// Z takes out_rows * out_cols * R*S*C floats per image: the caller's
// workspace when it is big enough for at least one image, else a
// stream-ordered temporary of up to 64 MiB; images go through in minibatches.
static int launch_input_backprop_col2im(const float* dy, const float* filter,
                                        float* dx,
                                        const snn_hip_conv2d_params& p,
                                        float* workspace,
                                        size_t workspace_elems,
                                        hipStream_t stream) {
  const int q_total = p.window_rows * p.window_cols * p.channels;
  const size_t z_per_image =
      static_cast<size_t>(p.out_rows) * p.out_cols * q_total;
  float* z = workspace;
  size_t z_elems = workspace_elems;
  bool temporary = false;
  if (z == nullptr || z_elems < z_per_image ||
      (reinterpret_cast<uintptr_t>(z) & 15u) != 0) {
    const size_t cap = max(z_per_image, (size_t{64} << 20) / sizeof(float));
    z_elems = min(cap, z_per_image * p.batch);
    void* ptr = nullptr;
    if (temp_malloc_async(&ptr, z_elems * sizeof(float), stream) != hipSuccess)
      return SNN_HIP_ALLOCATION_PROBLEM;
    z = static_cast<float*>(ptr);
    temporary = true;
  }
  // at most kMaxBufferBytes of Z per GEMM launch
  const size_t max_images = min(z_elems, kMaxBufferBytes / sizeof(float)) /
                            z_per_image;
  const int minibatch = static_cast<int>(
      max(size_t{1}, min(static_cast<size_t>(p.batch), max_images)));

  FilterBackpropGeom fg;
  fg.batch = p.batch; fg.in_rows = p.in_rows; fg.in_cols = p.in_cols;
  fg.channels = p.channels; fg.out_rows = p.out_rows; fg.out_cols = p.out_cols;
  fg.features = p.features; fg.win_rows = p.window_rows;
  fg.win_cols = p.window_cols; fg.stride_rows = p.stride_rows;
  fg.stride_cols = p.stride_cols; fg.pad_rows = p.pad_rows;
  fg.pad_cols = p.pad_cols; fg.m_total = 0;

  const size_t wgt_elems = static_cast<size_t>(q_total) * p.features;
  for (int first = 0; first < p.batch; first += minibatch) {
    const int images = min(minibatch, p.batch - first);
    Gather g;
    g.batch = images;
    g.p_rows = p.out_rows; g.p_cols = p.out_cols;
    g.src_rows = p.out_rows; g.src_cols = p.out_cols;
    g.src_ch = p.features;
    g.win_rows = g.win_cols = 1;
    g.step_rows = g.step_cols = 1;
    g.off_rows = g.off_cols = 0;
    g.tap_sign = 1;
    g.div_rows = g.div_cols = 1;
    g.m_total = images * p.out_rows * p.out_cols;
    g.k_total = p.features;
    g.n_total = q_total;
    g.z_src = g.z_wgt = g.z_dst = 0;
    const size_t dy_elems = static_cast<size_t>(g.m_total) * p.features;
    const float* dy_mb = dy + static_cast<size_t>(first) * p.out_rows *
                                  p.out_cols * p.features;
    launch_tile<64, 64, 2, 2, true, false>(dy_mb, filter, z, g, dy_elems,
                                           wgt_elems, 1, stream);
    const size_t dx_elems = static_cast<size_t>(images) * p.in_rows *
                            p.in_cols * p.channels;
    float* dx_mb = dx + static_cast<size_t>(first) * p.in_rows * p.in_cols *
                            p.channels;
    hipLaunchKernelGGL(col2im_gather_kernel,
                       dim3(static_cast<unsigned>(ceil_div(dx_elems, size_t{256}))),
                       dim3(256), 0, stream, z, dx_mb, fg, images);
  }
  const hipError_t err = hipGetLastError();
  if (temporary) temp_free_async(z, stream);
  if (err != hipSuccess) return report_hip_error(err, "input backprop col2im");
  return SNN_HIP_OK;
}

// Every shape it supports except those the one-work-group kernel takes (few
// (tap, channel) pairs, e.g. a three-channel stem).
bool conv2d_filter_backprop_direct_f32_wanted(const snn_hip_conv2d_params& p,
                                              bool reproducible) {
  const bool whole = p.channels % 64 == 0 && p.features % 64 == 0;
  // (from 32 channels on the 64-channel tiles are at least half full and
  // measured faster: 112x112x32 -> 64, 1x1, at batch 32 89.6 us there; with
  // at most eight channels they are so empty that the one-work-group kernel
  // in parts wins -- 11x11x3 -> 96 stride 4 at batch 16: 1000 us here -- but
  // it sums through atomics, so a reproducible launch stays here)
  const int q = p.window_rows * p.window_cols * p.channels;
  const bool small_q =
      p.features % 4 == 0 &&
      ((p.channels < 32 && q <= kSmallQMax) ||
       (!reproducible && p.channels <= kSmallQPartsMaxChannels &&
        q <= kSmallQParts * kSmallQMax));
  if (small_q || !conv2d_filter_backprop_direct_f32_supports(p, true))
    return false;
  return !whole || SNN_TUNING_ENV("SNN_HIP_FBDIRECT_OFF") == nullptr;
}

static int launch_filter_backprop(const float* x, const float* dy, float* dw,
                                  const snn_hip_conv2d_params& p,
                                  float* workspace, size_t workspace_elems,
                                  hipStream_t stream, bool reproducible) {
  FilterBackpropGeom g;
  g.batch = p.batch; g.in_rows = p.in_rows; g.in_cols = p.in_cols;
  g.channels = p.channels; g.out_rows = p.out_rows; g.out_cols = p.out_cols;
  g.features = p.features; g.win_rows = p.window_rows;
  g.win_cols = p.window_cols; g.stride_rows = p.stride_rows;
  g.stride_cols = p.stride_cols; g.pad_rows = p.pad_rows;
  g.pad_cols = p.pad_cols;
  g.m_total = p.batch * p.out_rows * p.out_cols;
  const size_t x_elems =
      static_cast<size_t>(p.batch) * p.in_rows * p.in_cols * p.channels;
  const size_t dy_elems = static_cast<size_t>(g.m_total) * p.features;
  const size_t dw_elems = static_cast<size_t>(p.window_rows) * p.window_cols *
                          p.channels * p.features;
  if (conv2d_stem_filter_backprop_supports(p) &&
      (reinterpret_cast<uintptr_t>(dw) & 15u) == 0 &&
      SNN_TUNING_ENV("SNN_HIP_STEM_OFF") == nullptr)
    return launch_conv2d_stem_filter_backprop_f32(x, dy, dw, p, stream);
  if (conv2d_filter_backprop_direct_f32_wanted(p, reproducible)) {
    // partial filters go to the workspace when it holds them, else to a
    // stream-ordered temporary
    const size_t part_floats = conv2d_filter_backprop_direct_f32_partial_floats(p);
    float* part = workspace;
    const bool own =
        part_floats != 0 &&
        (workspace == nullptr ||
         (reinterpret_cast<uintptr_t>(workspace) & 15u) != 0 ||
         workspace_elems < part_floats);
    if (own) {
      void* ptr = nullptr;
      if (temp_malloc_async(&ptr, part_floats * sizeof(float), stream) !=
          hipSuccess)
        return SNN_HIP_ALLOCATION_PROBLEM;
      part = static_cast<float*>(ptr);
    }
    const int status =
        launch_conv2d_filter_backprop_direct_f32(x, dy, dw, part, p, stream);
    const hipError_t err = hipGetLastError();
    if (own) temp_free_async(part, stream);
    if (status != SNN_HIP_OK) return status;
    if (err != hipSuccess) return report_hip_error(err, "filter backprop");
    return SNN_HIP_OK;
  }
  if (p.channels % 64 != 0) {
    // few (tap, channel) pairs: one work-group column per 64 features, the
    // pixel range split over about two work-groups per CU
    const int n_chunks = ceil_div(g.m_total, kBK);
    const int q_parts =
        ceil_div(p.window_rows * p.window_cols * p.channels, kSmallQMax);
    const int col_groups = ceil_div(p.features, 64);
    int splits =
        max(1, min(ceil_div(512, col_groups * q_parts), n_chunks / 4));
    const int per_split = ceil_div(n_chunks, splits);
    splits = ceil_div(n_chunks, per_split);
    const size_t n_vec = dw_elems / 4;  // features % 4 == 0
    hipLaunchKernelGGL(zero_fill_kernel,
                       dim3(static_cast<unsigned>(ceil_div(n_vec, size_t{256}))),
                       dim3(256), 0, stream, reinterpret_cast<float4*>(dw),
                       n_vec);
    constexpr size_t kLdsBytes =
        2 * sizeof(float) * (kBK * kSmallQStride + row_inner_floats(64));
    static const hipError_t attr = hipFuncSetAttribute(
        reinterpret_cast<const void*>(conv_filter_backprop_smallq_kernel),
        hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes);
    (void)attr;
    KernelTimer timer(stream);
    hipLaunchKernelGGL(conv_filter_backprop_smallq_kernel,
                       dim3(col_groups, splits, q_parts), dim3(kThreads),
                       kLdsBytes, stream, x, dy, dw, g, static_cast<unsigned>(x_elems * 4),
                       static_cast<unsigned>(dy_elems * 4),
                       static_cast<unsigned>(dw_elems * 4), per_split);
    return SNN_HIP_OK;
  }
  const int tiles = (p.window_rows * p.window_cols * p.channels / 64) *
                    ceil_div(p.features, 64);
  const int n_chunks = ceil_div(g.m_total, kBK);
  // (1x1 windows: half as many units measured 2-14 % faster on the four
  // batch-32 K = 4C layers, 3x3 windows up to 13 % slower on the deeper two)
  const int units =
      p.window_rows * p.window_cols == 1 ? kSplitUnits / 2 : kSplitUnits;
  int splits = max(1, min(ceil_div(units, tiles),
                          n_chunks / kMinChunksPerSplit));
  const int per_split = ceil_div(n_chunks, splits);
  splits = ceil_div(n_chunks, per_split);
  const size_t n_vec = dw_elems / 4;
  hipLaunchKernelGGL(zero_fill_kernel,
                     dim3(static_cast<unsigned>(ceil_div(n_vec, size_t{256}))),
                     dim3(256), 0, stream, reinterpret_cast<float4*>(dw), n_vec);
  KernelTimer timer(stream);
  hipLaunchKernelGGL(conv_filter_backprop_kernel<float>, dim3(tiles, splits),
                     dim3(kThreads), 0, stream, x, dy, dw, g,
                     static_cast<unsigned>(x_elems * 4),
                     static_cast<unsigned>(dy_elems * 4),
                     static_cast<unsigned>(dw_elems * 4), per_split);
  return SNN_HIP_OK;
}

namespace {

// dX of a strided 1x1 unpadded convolution from the dense gradient of its
// output pixels: dx[n][y][x][.] = t[n][y / sr][x / sc][.] where both
// coordinates are multiples of the strides (and the quotient is an output
// pixel), zero elsewhere.  One float4 per lane; every element of dX written.
__global__ void __launch_bounds__(256)
    scatter_strided_pixels_kernel(const float4* __restrict__ t,
                                  float4* __restrict__ dx, int in_rows,
                                  int in_cols, int out_rows, int out_cols,
                                  int stride_rows, int stride_cols, int cv,
                                  size_t n_vec) {
  const size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
  if (i >= n_vec) return;
  const int c = static_cast<int>(i % cv);
  size_t pix = i / cv;
  const int x = static_cast<int>(pix % in_cols);
  pix /= in_cols;
  const int y = static_cast<int>(pix % in_rows);
  const size_t n = pix / in_rows;
  const int oy = y / stride_rows, ox = x / stride_cols;
  float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
  if (oy * stride_rows == y && ox * stride_cols == x && oy < out_rows &&
      ox < out_cols)
    v = t[((n * out_rows + oy) * out_cols + ox) * cv + c];
  dx[i] = v;
}

// Strided input gradient by stride classes.  The input pixels whose
// coordinates are (py, px) modulo the strides receive gradient only through
// the taps r = rho_r + sr u, s = rho_s + sc v with rho = (p + pad) mod stride,
// and for them the gradient is a stride-1 convolution of dY with that
// sub-filter, channels and features exchanged:
//   dX[n][sr y' + py][sc x' + px][c] =
//       sum_{u', v', k} dY[n][y' - pad'_r + u'][x' - pad'_c + v'][k] G[u'][v'][k][c]
// with G[u'][v'][k][c] = W[rho_r + sr (Rc - 1 - u')][rho_s + sc (Sc - 1 - v')][c][k]
// and pad' = Rc - 1 - (p + pad - rho) / stride.
constexpr int kMaxStrideClasses = 16;
struct StrideClasses {
  int stride_rows, stride_cols, pad_rows, pad_cols;
  int win_rows, win_cols, channels, features;
  // per class (py * stride_cols + px): first element of its sub-filter and
  // of its dense result, its size in pixels
  unsigned filter_base[kMaxStrideClasses];
  size_t pixel_base[kMaxStrideClasses];  // in units of pixels (x channels)
  int rows[kMaxStrideClasses], cols[kMaxStrideClasses];
  int taps_r[kMaxStrideClasses], taps_c[kMaxStrideClasses];
};

// Every filter element to its place in the sub-filter of its class: per tap
// a C x K matrix becomes K x C, 32 x 32 tiles through LDS so that reads and
// writes are both contiguous.  Grid: (K tiles, C tiles, taps), 32 x 8 lanes.
template <typename T>
__global__ void __launch_bounds__(256)
    stride_class_filters_kernel(const T* __restrict__ w, T* __restrict__ g,
                                StrideClasses sc) {
  __shared__ T tile[32][33];
  const int tap = blockIdx.z;
  const int s = tap % sc.win_cols;
  const int r = tap / sc.win_cols;
  const int py = ((r - sc.pad_rows) % sc.stride_rows + sc.stride_rows) %
                 sc.stride_rows;
  const int px = ((s - sc.pad_cols) % sc.stride_cols + sc.stride_cols) %
                 sc.stride_cols;
  const int cls = py * sc.stride_cols + px;
  if (sc.taps_r[cls] == 0) return;  // a class without pixels keeps no filter
  const int u = sc.taps_r[cls] - 1 - r / sc.stride_rows;  // r = rho + sr u
  const int v = sc.taps_c[cls] - 1 - s / sc.stride_cols;
  const int k0 = blockIdx.x * 32, c0 = blockIdx.y * 32;
  const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
  const T* const src =
      w + static_cast<size_t>(tap) * sc.channels * sc.features;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int c = c0 + ty + 8 * i, k = k0 + tx;
    tile[ty + 8 * i][tx] = (c < sc.channels && k < sc.features)
                               ? src[static_cast<size_t>(c) * sc.features + k]
                               : static_cast<T>(0);
  }
  __syncthreads();
  T* const dst =
      g + sc.filter_base[cls] +
      static_cast<size_t>(u * sc.taps_c[cls] + v) * sc.features * sc.channels;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int k = k0 + ty + 8 * i, c = c0 + tx;
    if (k < sc.features && c < sc.channels)
      dst[static_cast<size_t>(k) * sc.channels + c] = tile[tx][ty + 8 * i];
  }
}

// dX from the dense results of the classes (zeros for a class no tap reaches).
template <typename V>  // four elements: float4, or 8 bytes of binary16
__global__ void __launch_bounds__(256)
    interleave_stride_classes_kernel(const V* __restrict__ t,
                                     V* __restrict__ dx, StrideClasses sc,
                                     int in_rows, int in_cols, int cv,
                                     size_t n_vec) {
  const size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
  if (i >= n_vec) return;
  const int c = static_cast<int>(i % cv);
  size_t pix = i / cv;
  const int x = static_cast<int>(pix % in_cols);
  pix /= in_cols;
  const int y = static_cast<int>(pix % in_rows);
  const size_t n = pix / in_rows;
  const int cls = (y % sc.stride_rows) * sc.stride_cols + x % sc.stride_cols;
  V v = {};
  if (sc.taps_r[cls] > 0 && sc.taps_c[cls] > 0)
    v = t[(sc.pixel_base[cls] +
           (n * sc.rows[cls] + y / sc.stride_rows) * sc.cols[cls] +
           x / sc.stride_cols) * cv + c];
  dx[i] = v;
}

__global__ void __launch_bounds__(256)
    f32_to_f16_kernel(const float* __restrict__ in, _Float16* __restrict__ out,
                      size_t n) {
  const size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
  if (i < n) out[i] = static_cast<_Float16>(in[i]);
}

void fill_gather(const snn_hip_conv2d_params& p, int direction, Gather* g) {
  g->batch = p.batch;
  g->win_rows = p.window_rows;
  g->win_cols = p.window_cols;
  if (direction == SNN_HIP_FORWARD) {
    g->p_rows = p.out_rows;  g->p_cols = p.out_cols;
    g->src_rows = p.in_rows; g->src_cols = p.in_cols;
    g->src_ch = p.channels;
    g->step_rows = p.stride_rows; g->step_cols = p.stride_cols;
    g->off_rows = -p.pad_rows;    g->off_cols = -p.pad_cols;
    g->tap_sign = 1;
    g->div_rows = g->div_cols = 1;
    g->n_total = p.features;
  } else {
    g->p_rows = p.in_rows;    g->p_cols = p.in_cols;
    g->src_rows = p.out_rows; g->src_cols = p.out_cols;
    g->src_ch = p.features;
    g->step_rows = g->step_cols = 1;
    g->off_rows = p.pad_rows; g->off_cols = p.pad_cols;
    g->tap_sign = -1;
    g->div_rows = p.stride_rows; g->div_cols = p.stride_cols;
    g->n_total = p.channels;
  }
  g->m_total = g->batch * g->p_rows * g->p_cols;
  g->k_total = g->win_rows * g->win_cols * g->src_ch;
  g->z_src = g->z_wgt = g->z_dst = 0;
}

}  // namespace

// Half-precision filter gradient on the matrix cores: the fp32 kernel reads
// binary16 operands (converted on the way into LDS, so every product and sum
// is what an f16 matrix instruction with fp32 accumulation would give),
// accumulates dW in an fp32 buffer -- the workspace when it holds 2 * R*S*C*K
// halves, else a stream-ordered temporary -- and one pass rounds it to
// binary16.
bool conv2d_filter_backprop_f16_supports(const snn_hip_conv2d_params& p) {
  const size_t x = static_cast<size_t>(p.batch) * p.in_rows * p.in_cols *
                   p.channels;
  const size_t y = static_cast<size_t>(p.batch) * p.out_rows * p.out_cols *
                   p.features;
  return (p.channels % 64 == 0 && p.features % 4 == 0 &&
          max(x, y) * sizeof(_Float16) <= kMaxBufferBytes &&
          static_cast<size_t>(p.window_rows) * p.window_cols * p.channels *
                  p.features * sizeof(float) <= kMaxBufferBytes) ||
         conv2d_filter_backprop_direct_f16_supports(p);
}

int launch_conv2d_filter_backprop_f16(const _Float16* x, const _Float16* dy,
                                      _Float16* dw,
                                      const snn_hip_conv2d_params& p,
                                      _Float16* workspace,
                                      size_t workspace_elems,
                                      hipStream_t stream) {
  FilterBackpropGeom g;
  g.batch = p.batch; g.in_rows = p.in_rows; g.in_cols = p.in_cols;
  g.channels = p.channels; g.out_rows = p.out_rows; g.out_cols = p.out_cols;
  g.features = p.features; g.win_rows = p.window_rows;
  g.win_cols = p.window_cols; g.stride_rows = p.stride_rows;
  g.stride_cols = p.stride_cols; g.pad_rows = p.pad_rows;
  g.pad_cols = p.pad_cols;
  g.m_total = p.batch * p.out_rows * p.out_cols;
  const size_t x_elems =
      static_cast<size_t>(p.batch) * p.in_rows * p.in_cols * p.channels;
  const size_t dy_elems = static_cast<size_t>(g.m_total) * p.features;
  const size_t dw_elems = static_cast<size_t>(p.window_rows) * p.window_cols *
                          p.channels * p.features;
  const bool ws_aligned =
      workspace != nullptr && (reinterpret_cast<uintptr_t>(workspace) & 15u) == 0;
  const bool is_3x3 = conv2d_filter_backprop_3x3_f16_supports(p);
  if ((is_3x3 || conv2d_filter_backprop_1x1_f16_supports(p)) &&
      (reinterpret_cast<uintptr_t>(dw) & 7u) == 0 &&
      SNN_TUNING_ENV("SNN_HIP_FILBK_F16_OFF") == nullptr) {
    // binary16 matrix instructions; the partial tiles go to the workspace
    // when it holds them, else to a stream-ordered temporary
    const size_t part_floats =
        is_3x3 ? conv2d_filter_backprop_3x3_f16_partial_floats(p)
               : conv2d_filter_backprop_1x1_f16_partial_floats(p);
    float* part = reinterpret_cast<float*>(workspace);
    const bool own = !ws_aligned || workspace_elems < 2 * part_floats;
    if (own) {
      void* ptr = nullptr;
      if (temp_malloc_async(&ptr, part_floats * sizeof(float), stream) !=
          hipSuccess)
        return SNN_HIP_ALLOCATION_PROBLEM;
      part = static_cast<float*>(ptr);
    }
    const int status =
        is_3x3
            ? launch_conv2d_filter_backprop_3x3_f16(x, dy, dw, part, p, stream)
            : launch_conv2d_filter_backprop_1x1_f16(x, dy, dw, part, p, stream);
    const hipError_t err = hipGetLastError();
    if (own) temp_free_async(part, stream);
    if (status != SNN_HIP_OK) return status;
    if (err != hipSuccess) return report_hip_error(err, "f16 filter backprop");
    return SNN_HIP_OK;
  }
  if (conv2d_filter_backprop_direct_f16_supports(p)) {
    // every other shape with at least 256 output pixels: binary16 operands
    // converted on the way into the fp32 matrix instruction's registers, fp32
    // partial filters (workspace or temporary), one pass that adds and rounds
    const size_t part_floats = conv2d_filter_backprop_direct_f16_partial_floats(p);
    float* part = reinterpret_cast<float*>(workspace);
    const bool own = !ws_aligned || workspace_elems < 2 * part_floats;
    if (own) {
      void* ptr = nullptr;
      if (temp_malloc_async(&ptr, part_floats * sizeof(float), stream) !=
          hipSuccess)
        return SNN_HIP_ALLOCATION_PROBLEM;
      part = static_cast<float*>(ptr);
    }
    const int status =
        launch_conv2d_filter_backprop_direct_f16(x, dy, dw, part, p, stream);
    const hipError_t err = hipGetLastError();
    if (own) temp_free_async(part, stream);
    if (status != SNN_HIP_OK) return status;
    if (err != hipSuccess) return report_hip_error(err, "f16 filter backprop");
    return SNN_HIP_OK;
  }
  float* acc32 = reinterpret_cast<float*>(workspace);
  bool temporary = false;
  if (workspace == nullptr || workspace_elems < 2 * dw_elems ||
      (reinterpret_cast<uintptr_t>(workspace) & 15u) != 0) {
    void* ptr = nullptr;
    if (temp_malloc_async(&ptr, dw_elems * sizeof(float), stream) != hipSuccess)
      return SNN_HIP_ALLOCATION_PROBLEM;
    acc32 = static_cast<float*>(ptr);
    temporary = true;
  }
  const int tiles = (p.window_rows * p.window_cols * p.channels / 64) *
                    ceil_div(p.features, 64);
  const int n_chunks = ceil_div(g.m_total, kBK);
  int splits = max(1, min(ceil_div(kSplitUnits, tiles),
                          n_chunks / kMinChunksPerSplit));
  const int per_split = ceil_div(n_chunks, splits);
  splits = ceil_div(n_chunks, per_split);
  const size_t n_vec = dw_elems / 4;
  hipLaunchKernelGGL(zero_fill_kernel,
                     dim3(static_cast<unsigned>(ceil_div(n_vec, size_t{256}))),
                     dim3(256), 0, stream, reinterpret_cast<float4*>(acc32),
                     n_vec);
  {
    KernelTimer timer(stream);
    hipLaunchKernelGGL(conv_filter_backprop_kernel<_Float16>,
                       dim3(tiles, splits), dim3(kThreads), 0, stream, x, dy,
                       acc32, g, static_cast<unsigned>(x_elems * 2),
                       static_cast<unsigned>(dy_elems * 2),
                       static_cast<unsigned>(dw_elems * 4), per_split);
  }
  hipLaunchKernelGGL(f32_to_f16_kernel,
                     dim3(static_cast<unsigned>(ceil_div(dw_elems, size_t{256}))),
                     dim3(256), 0, stream, acc32, dw, dw_elems);
  const hipError_t err = hipGetLastError();
  if (temporary) temp_free_async(acc32, stream);
  if (err != hipSuccess) return report_hip_error(err, "f16 filter backprop");
  return SNN_HIP_OK;
}

// Half-precision input gradient for the shapes the LDS-tile kernel does not
// take (strides, channel counts that are not multiples of 64): the general
// implicit-GEMM kernel reading binary16 operands, one work-group per 64 x 64
// tile of dX and no reduction split, so every output is stored once.
bool conv2d_input_backprop_general_f16_supports(
    const snn_hip_conv2d_params& p) {
  const size_t x = static_cast<size_t>(p.batch) * p.in_rows * p.in_cols *
                   p.channels;
  const size_t y = static_cast<size_t>(p.batch) * p.out_rows * p.out_cols *
                   p.features;
  const size_t w = static_cast<size_t>(p.window_rows) * p.window_cols *
                   p.channels * p.features;
  return p.features % 4 == 0 &&
         max(max(x, y), w) * sizeof(_Float16) <= kMaxBufferBytes;
}

int launch_conv2d_input_backprop_general_f16(const _Float16* dy,
                                             const _Float16* filter,
                                             _Float16* dx,
                                             const snn_hip_conv2d_params& p,
                                             hipStream_t stream) {
  Gather g;
  fill_gather(p, SNN_HIP_INPUT_BACKPROP, &g);
  constexpr int BM = 64, BN = 64;
  const unsigned tiles_m = static_cast<unsigned>(ceil_div(g.m_total, BM));
  const unsigned tiles_n = static_cast<unsigned>(ceil_div(g.n_total, BN));
  const unsigned n_tiles = tiles_m * tiles_n;
  const int n_chunks = ceil_div(g.k_total, kBK);
  constexpr size_t kLdsBytes =
      2 * sizeof(float) * (k_inner_floats(BM) + k_inner_floats(BN));
  const unsigned src_bytes = static_cast<unsigned>(
      static_cast<size_t>(g.batch) * g.src_rows * g.src_cols * g.src_ch * 2);
  const unsigned wgt_bytes = static_cast<unsigned>(
      static_cast<size_t>(p.window_rows) * p.window_cols * p.channels *
      p.features * 2);
  KernelTimer timer(stream);
  if (g.div_rows != 1 || g.div_cols != 1) {
    hipLaunchKernelGGL(
        (conv_igemm_kernel<BM, BN, 2, 2, true, true, false, false, _Float16>),
        dim3(n_tiles, 1), dim3(kThreads), kLdsBytes, stream, dy, filter, dx, g,
        src_bytes, wgt_bytes, tiles_n, n_tiles, n_chunks);
  } else {
    hipLaunchKernelGGL(
        (conv_igemm_kernel<BM, BN, 2, 2, true, false, false, false, _Float16>),
        dim3(n_tiles, 1), dim3(kThreads), kLdsBytes, stream, dy, filter, dx, g,
        src_bytes, wgt_bytes, tiles_n, n_tiles, n_chunks);
  }
  SNN_HIP_CHECK_LAUNCH();
  return SNN_HIP_OK;
}

// Half-precision forward convolution for the shapes the binary16 kernels do
// not take (channel counts that are not multiples of 64, windows of more than
// 32 taps): the same general kernel, gathering X four channels at a time.
bool conv2d_forward_general_f16_supports(const snn_hip_conv2d_params& p) {
  const size_t x = static_cast<size_t>(p.batch) * p.in_rows * p.in_cols *
                   p.channels;
  const size_t y = static_cast<size_t>(p.batch) * p.out_rows * p.out_cols *
                   p.features;
  const size_t w = static_cast<size_t>(p.window_rows) * p.window_cols *
                   p.channels * p.features;
  return p.channels % 4 == 0 && p.features % 4 == 0 &&
         max(max(x, y), w) * sizeof(_Float16) <= kMaxBufferBytes;
}

int launch_conv2d_forward_general_f16(const _Float16* x, const _Float16* filter,
                                      _Float16* y,
                                      const snn_hip_conv2d_params& p,
                                      hipStream_t stream) {
  Gather g;
  fill_gather(p, SNN_HIP_FORWARD, &g);
  constexpr int BM = 64, BN = 64;
  const unsigned tiles_m = static_cast<unsigned>(ceil_div(g.m_total, BM));
  const unsigned tiles_n = static_cast<unsigned>(ceil_div(g.n_total, BN));
  const unsigned n_tiles = tiles_m * tiles_n;
  const int n_chunks = ceil_div(g.k_total, kBK);
  constexpr size_t kLdsBytes =
      2 * sizeof(float) * (k_inner_floats(BM) + row_inner_floats(BN));
  const unsigned src_bytes = static_cast<unsigned>(
      static_cast<size_t>(g.batch) * g.src_rows * g.src_cols * g.src_ch * 2);
  const unsigned wgt_bytes = static_cast<unsigned>(
      static_cast<size_t>(p.window_rows) * p.window_cols * p.channels *
      p.features * 2);
  KernelTimer timer(stream);
  hipLaunchKernelGGL(
      (conv_igemm_kernel<BM, BN, 2, 2, false, false, false, false, _Float16>),
      dim3(n_tiles, 1), dim3(kThreads), kLdsBytes, stream, x, filter, y, g,
      src_bytes, wgt_bytes, tiles_n, n_tiles, n_chunks);
  SNN_HIP_CHECK_LAUNCH();
  return SNN_HIP_OK;
}

bool conv2d_igemm_supports(int direction, const snn_hip_conv2d_params& p) {
  // buffer descriptors address at most kMaxBufferBytes
  const size_t x = static_cast<size_t>(p.batch) * p.in_rows * p.in_cols *
                   p.channels;
  const size_t y = static_cast<size_t>(p.batch) * p.out_rows * p.out_cols *
                   p.features;
  const size_t w = static_cast<size_t>(p.window_rows) * p.window_cols *
                   p.channels * p.features;
  if (max(max(x, y), w) * sizeof(float) > kMaxBufferBytes) return false;
  if (direction == SNN_HIP_FORWARD) return p.features % 4 == 0;
  if (direction == SNN_HIP_INPUT_BACKPROP)
    return p.features % 4 == 0;
  // filter backprop: a 64-wide tile of (tap, channel) must lie inside one
  // tap, or the whole (tap, channel) range must fit one work-group
  return (p.features % 4 == 0 &&
          (p.channels % 64 == 0 ||
           p.window_rows * p.window_cols * p.channels <= kSmallQMax)) ||
         conv2d_filter_backprop_direct_f32_supports(p, true);
}

bool batched_gemm_mfma_supports(int m, int k, int n, const void* a,
                                const void* b, const void* c,
                                bool transpose_b) {
  auto aligned = [](const void* p) {
    return (reinterpret_cast<uintptr_t>(p) & 15u) == 0;
  };
  return k % kBK == 0 && (transpose_b || n % 4 == 0) && aligned(a) &&
         aligned(b) && aligned(c) &&
         static_cast<size_t>(m) * max(k, n) * sizeof(float) <= kMaxBufferBytes &&
         static_cast<size_t>(k) * n * sizeof(float) <= kMaxBufferBytes;
}

int launch_batched_gemm_mfma_f32(const float* a, const float* b, float* c,
                                 int batches, int m, int k, int n,
                                 hipStream_t stream, bool transpose_b,
                                 bool accumulate, bool deterministic) {
  // C[z] (+)= A[z] (m x k) * op(B[z]): a 1x1 "convolution" over m pixels.  B
  // as k x n is the forward filter layout, B as n x k (transpose_b) the
  // K-contiguous layout of the input-gradient kernel.
  Gather g;
  g.batch = 1;
  g.p_rows = 1; g.p_cols = m;
  g.src_rows = 1; g.src_cols = m;
  g.src_ch = k;
  g.win_rows = g.win_cols = 1;
  g.step_rows = g.step_cols = 1;
  g.off_rows = g.off_cols = 0;
  g.tap_sign = 1;
  g.div_rows = g.div_cols = 1;
  g.m_total = m;
  g.k_total = k;
  g.n_total = n;
  g.z_src = m * k;
  g.z_wgt = k * n;
  g.z_dst = m * n;
  const long tiles = static_cast<long>(ceil_div(m, 64)) * ceil_div(n, 64) * batches;
  const int n_chunks = k / kBK;
  int splits = 1;
  // the zero fill of a split launch writes float4s
  const bool can_split =
      accumulate || (static_cast<size_t>(batches) * m * n) % 4 == 0;
  if (tiles < kResidentSlots && can_split && !deterministic) {
    splits = static_cast<int>((kSplitUnits + tiles - 1) / tiles);
    splits = max(1, min(splits, n_chunks / kMinChunksPerSplit));
  }
  if (!transpose_b && !accumulate && gemm_rows_wanted(m, k, n, batches)) {
    launch_gemm_rows(a, b, c, m, k, n, batches, m * k, k * n, m * n, stream,
                     nullptr);
    SNN_HIP_CHECK_LAUNCH();
    return SNN_HIP_OK;
  }
  if (transpose_b)
    launch_tile<64, 64, 2, 2, true, false>(a, b, c, g,
                                           static_cast<size_t>(m) * k,
                                           static_cast<size_t>(k) * n, splits,
                                           stream, batches, accumulate);
  else
    launch_tile<64, 64, 2, 2, false, false>(a, b, c, g,
                                            static_cast<size_t>(m) * k,
                                            static_cast<size_t>(k) * n, splits,
                                            stream, batches, accumulate);
  SNN_HIP_CHECK_LAUNCH();
  return SNN_HIP_OK;
}

// The stride classes of an input gradient, each through `forward` (a
// stride-1 forward convolution of T tensors: parameters, input, filter,
// output), then interleaved.  Returns -1 when a class would need negative
// padding (the caller then takes another path).
template <typename T, typename V, typename Forward>
int strided_input_backprop_by_classes(const T* input, const T* filter,
                                      T* output,
                                      const snn_hip_conv2d_params& p,
                                      hipStream_t stream, Forward forward) {
  StrideClasses sc;
  sc.stride_rows = p.stride_rows; sc.stride_cols = p.stride_cols;
  sc.pad_rows = p.pad_rows;       sc.pad_cols = p.pad_cols;
  sc.win_rows = p.window_rows;    sc.win_cols = p.window_cols;
  sc.channels = p.channels;       sc.features = p.features;
  bool ok = true;
  unsigned filter_elems = 0;
  size_t pixels = 0;
  int pad_r[kMaxStrideClasses], pad_c[kMaxStrideClasses];
  for (int py = 0; py < p.stride_rows; ++py)
    for (int px = 0; px < p.stride_cols; ++px) {
      const int cls = py * p.stride_cols + px;
      const int rho_r = (py + p.pad_rows) % p.stride_rows;
      const int rho_c = (px + p.pad_cols) % p.stride_cols;
      sc.taps_r[cls] =
          max(0, (p.window_rows - rho_r + p.stride_rows - 1) / p.stride_rows);
      sc.taps_c[cls] =
          max(0, (p.window_cols - rho_c + p.stride_cols - 1) / p.stride_cols);
      sc.rows[cls] = max(0, (p.in_rows - py + p.stride_rows - 1) / p.stride_rows);
      sc.cols[cls] = max(0, (p.in_cols - px + p.stride_cols - 1) / p.stride_cols);
      pad_r[cls] = sc.taps_r[cls] - 1 - (py + p.pad_rows - rho_r) / p.stride_rows;
      pad_c[cls] = sc.taps_c[cls] - 1 - (px + p.pad_cols - rho_c) / p.stride_cols;
      sc.filter_base[cls] = filter_elems;
      sc.pixel_base[cls] = pixels;
      const bool empty = sc.taps_r[cls] == 0 || sc.taps_c[cls] == 0 ||
                         sc.rows[cls] == 0 || sc.cols[cls] == 0;
      if (!empty) {
        ok = ok && pad_r[cls] >= 0 && pad_c[cls] >= 0;
        pixels += static_cast<size_t>(p.batch) * sc.rows[cls] * sc.cols[cls];
      } else {
        sc.taps_r[cls] = sc.taps_c[cls] = 0;
      }
      filter_elems += static_cast<unsigned>(sc.taps_r[cls]) * sc.taps_c[cls] *
                      p.channels * p.features;
    }
  if (ok) {
    void *g = nullptr, *t = nullptr;
    // (no room for the temporaries: the caller takes another path)
    if (temp_malloc_async(&g, max(filter_elems, 4u) * sizeof(T), stream) !=
        hipSuccess) {
      (void)hipGetLastError();
      return -1;
    }
    if (temp_malloc_async(&t, max(pixels, size_t{1}) * p.channels * sizeof(T),
                          stream) != hipSuccess) {
      (void)hipGetLastError();
      temp_free_async(g, stream);
      return -1;
    }
    hipLaunchKernelGGL(
        stride_class_filters_kernel<T>,
        dim3(static_cast<unsigned>(ceil_div(p.features, 32)),
             static_cast<unsigned>(ceil_div(p.channels, 32)),
             static_cast<unsigned>(p.window_rows * p.window_cols)),
        dim3(256), 0, stream, filter, static_cast<T*>(g), sc);
    int status = SNN_HIP_OK;
    for (int cls = 0; cls < p.stride_rows * p.stride_cols; ++cls) {
      if (sc.taps_r[cls] == 0 || status != SNN_HIP_OK) continue;
      snn_hip_conv2d_params q = p;
      q.in_rows = p.out_rows;   q.in_cols = p.out_cols;
      q.out_rows = sc.rows[cls]; q.out_cols = sc.cols[cls];
      q.channels = p.features;  q.features = p.channels;
      q.window_rows = sc.taps_r[cls]; q.window_cols = sc.taps_c[cls];
      q.stride_rows = q.stride_cols = 1;
      q.pad_rows = pad_r[cls];  q.pad_cols = pad_c[cls];
      status = forward(q, input, static_cast<const T*>(g) + sc.filter_base[cls],
                       static_cast<T*>(t) + sc.pixel_base[cls] * p.channels);
    }
    if (status == SNN_HIP_OK) {
      const size_t n_vec = static_cast<size_t>(p.batch) * p.in_rows *
                           p.in_cols * p.channels / 4;
      hipLaunchKernelGGL(
          interleave_stride_classes_kernel<V>,
          dim3(static_cast<unsigned>(ceil_div(n_vec, size_t{256}))),
          dim3(256), 0, stream, static_cast<const V*>(t),
          reinterpret_cast<V*>(output), sc, p.in_rows, p.in_cols,
          p.channels / 4, n_vec);
    }
    const hipError_t err = hipGetLastError();
    temp_free_async(t, stream);
    temp_free_async(g, stream);
    if (status != SNN_HIP_OK) return status;
    if (err != hipSuccess)
      return report_hip_error(err, "strided input backprop");
    return SNN_HIP_OK;
  }
  return -1;
}

bool conv2d_strided_input_backprop_f16_supports(
    const snn_hip_conv2d_params& p) {
  return (p.stride_rows > 1 || p.stride_cols > 1) &&
         p.stride_rows * p.stride_cols <= kMaxStrideClasses &&
         p.channels % 4 == 0 && p.features % 64 == 0 &&
         static_cast<double>(p.batch) * p.out_rows * p.out_cols *
                 p.window_rows * p.window_cols * p.channels * p.features >=
             double(1 << 30);
}

// Binary16: the classes run on the binary16 forward kernels (dY's feature
// count, the classes' channel count, in multiples of 64).  -1: not taken.
int launch_conv2d_strided_input_backprop_f16(const _Float16* dy,
                                             const _Float16* filter,
                                             _Float16* dx,
                                             const snn_hip_conv2d_params& p,
                                             hipStream_t stream) {
  typedef _Float16 half4v __attribute__((ext_vector_type(4)));
  return strided_input_backprop_by_classes<_Float16, half4v>(
      dy, filter, dx, p, stream,
      [&](const snn_hip_conv2d_params& q, const _Float16* in,
          const _Float16* fil, _Float16* out) {
        if (conv2d_igemm_f16_supports(q))
          return launch_conv2d_igemm_f16(in, fil, out, q, nullptr, 0, stream);
        return launch_conv2d_forward_general_f16(in, fil, out, q, stream);
      });
}

int launch_conv2d_igemm_f32(int direction, const float* input,
                            const float* filter, float* output,
                            const snn_hip_conv2d_params& p,
                            hipStream_t stream, float* workspace,
                            size_t workspace_elems,
                            const LaunchOptions* epilogue) {
  if (direction == SNN_HIP_FORWARD && conv2d_small_supports(p) &&
      SNN_TUNING_ENV("SNN_HIP_SMALL_OFF") == nullptr)
    return launch_conv2d_small_f32(input, filter, output, p, stream, epilogue);
  const bool aligned16 =
      ((reinterpret_cast<uintptr_t>(input) | reinterpret_cast<uintptr_t>(filter) |
        reinterpret_cast<uintptr_t>(output)) & 15u) == 0;
  if (direction == SNN_HIP_FORWARD && aligned16 &&
      conv2d_rowtile_supports(p) &&
      SNN_TUNING_ENV("SNN_HIP_ROWTILE_OFF") == nullptr)
    return launch_conv2d_rowtile_f32(input, filter, output, p, stream, false,
                                     epilogue);
  if (direction == SNN_HIP_FORWARD && aligned16 &&
      conv2d_rowsplit_supports(p) &&
      SNN_TUNING_ENV("SNN_HIP_ROWSPLIT_OFF") == nullptr)
    return launch_conv2d_rowsplit_f32(input, filter, output, p, stream, false,
                                      epilogue);
  if (direction == SNN_HIP_INPUT_BACKPROP && aligned16 &&
      p.window_rows == 1 && p.window_cols == 1 && p.pad_rows == 0 &&
      p.pad_cols == 0 && (p.stride_rows > 1 || p.stride_cols > 1) &&
      p.channels % 4 == 0 && p.features % 4 == 0 &&
      static_cast<size_t>(p.batch) * p.out_rows * p.out_cols >= 1024 &&
      SNN_TUNING_ENV("SNN_HIP_STRIDED_1X1_OFF") == nullptr) {
    // A strided 1x1 layer (a ResNet shortcut): only the input pixels at
    // multiples of the stride receive a gradient, and theirs is the stride-1
    // input gradient over the output pixels.  That product runs dense into a
    // stream-ordered temporary on the stride-1 kernels, and one pass writes
    // dX from it, zeros included (the general strided kernel multiplied the
    // zeros too: 56x56x256 -> 512 at batch 32 288 us).
    snn_hip_conv2d_params q = p;
    q.in_rows = p.out_rows;
    q.in_cols = p.out_cols;
    q.stride_rows = q.stride_cols = 1;
    const size_t t_elems =
        static_cast<size_t>(p.batch) * p.out_rows * p.out_cols * p.channels;
    void* t = nullptr;
    if (temp_malloc_async(&t, t_elems * sizeof(float), stream) == hipSuccess) {
      const int status = launch_conv2d_igemm_f32(
          direction, input, filter, static_cast<float*>(t), q, stream,
          workspace, workspace_elems, epilogue);
      if (status == SNN_HIP_OK) {
        const size_t n_vec = static_cast<size_t>(p.batch) * p.in_rows *
                             p.in_cols * p.channels / 4;
        hipLaunchKernelGGL(
            scatter_strided_pixels_kernel,
            dim3(static_cast<unsigned>(ceil_div(n_vec, size_t{256}))),
            dim3(256), 0, stream, static_cast<const float4*>(t),
            reinterpret_cast<float4*>(output), p.in_rows, p.in_cols,
            p.out_rows, p.out_cols, p.stride_rows, p.stride_cols,
            p.channels / 4, n_vec);
      }
      const hipError_t err = hipGetLastError();
      temp_free_async(t, stream);
      if (status != SNN_HIP_OK) return status;
      if (err != hipSuccess)
        return report_hip_error(err, "strided 1x1 input backprop");
      return SNN_HIP_OK;
    }
    (void)hipGetLastError();  // no room: the general strided kernel below
  }
  if (direction == SNN_HIP_INPUT_BACKPROP && aligned16 &&
      (p.stride_rows > 1 || p.stride_cols > 1) &&
      p.stride_rows * p.stride_cols <= kMaxStrideClasses &&
      p.channels % 4 == 0 && p.features % 4 == 0 &&
      // (from 2^30 multiply-adds: below that the extra launches cost more
      // than the multiplied zeros, 73 against 56 us at batch 4)
      static_cast<double>(p.batch) * p.out_rows * p.out_cols * p.window_rows *
              p.window_cols * p.channels * p.features >= double(1 << 30) &&
      SNN_TUNING_ENV("SNN_HIP_STRIDE_CLASSES_OFF") == nullptr) {
    // The general strided kernel walks every tap for every input pixel and
    // multiplies zeros for those that do not reach it (3/4 of them at stride
    // 2: 56x56x128 -> 128, 3x3, at batch 32 343 us against 90 forward).  By
    // stride classes every class is a dense stride-1 forward convolution of
    // dY on the fast kernels.
    const int rc = strided_input_backprop_by_classes<float, float4>(
        input, filter, output, p, stream,
        [&](const snn_hip_conv2d_params& q, const float* in, const float* fil,
            float* out) {
          return launch_conv2d_igemm_f32(SNN_HIP_FORWARD, in, fil, out, q, stream,
                                         nullptr, 0, nullptr);
        });
    if (rc >= 0) return rc;
  }
  if (direction == SNN_HIP_INPUT_BACKPROP && aligned16 &&
      p.stride_rows == 1 && p.stride_cols == 1 &&
      p.window_rows - 1 - p.pad_rows >= 0 &&
      p.window_cols - 1 - p.pad_cols >= 0 &&
      SNN_TUNING_ENV("SNN_HIP_ROWTILE_OFF") == nullptr) {
    // dX = dY convolved with the mirrored filter, channels and features
    // exchanged, padding window - 1 - pad
    snn_hip_conv2d_params q = p;
    q.in_rows = p.out_rows;   q.in_cols = p.out_cols;
    q.out_rows = p.in_rows;   q.out_cols = p.in_cols;
    q.channels = p.features;  q.features = p.channels;
    q.pad_rows = p.window_rows - 1 - p.pad_rows;
    q.pad_cols = p.window_cols - 1 - p.pad_cols;
    if (conv2d_rowtile_supports(q))
      return launch_conv2d_rowtile_f32(input, filter, output, q, stream, true,
                                       nullptr);
    if (conv2d_rowsplit_supports(q) &&
        SNN_TUNING_ENV("SNN_HIP_ROWSPLIT_OFF") == nullptr)
      return launch_conv2d_rowsplit_f32(input, filter, output, q, stream, true,
                                        nullptr);
  }
  if (direction == SNN_HIP_INPUT_BACKPROP &&
      conv2d_stem_input_backprop_supports(p) &&
      (reinterpret_cast<uintptr_t>(output) & 15u) == 0 &&
      (epilogue == nullptr || !epilogue->deterministic ||
       conv2d_stem_input_backprop_reproducible(p)) &&
      SNN_TUNING_ENV("SNN_HIP_STEM_OFF") == nullptr) {
    // three channels, 7x7 stride 2, 64 features: the kernel built for it
    return launch_conv2d_stem_input_backprop_f32(input, filter, output, p,
                                                 stream);
  }
  if (direction == SNN_HIP_INPUT_BACKPROP && p.channels < 16 &&
      p.features % kBK == 0 &&
      static_cast<size_t>(p.out_rows) * p.out_cols * p.window_rows *
              p.window_cols * p.channels * sizeof(float) <= kMaxBufferBytes)
    return launch_input_backprop_col2im(input, filter, output, p, workspace,
                                        workspace_elems, stream);
  if (direction == SNN_HIP_FILTER_BACKPROP) {
    const int rc = launch_filter_backprop(
        input, filter, output, p, workspace, workspace_elems, stream,
        epilogue != nullptr && epilogue->deterministic);
    SNN_HIP_CHECK_LAUNCH();
    return rc;
  }
  Gather g;
  g.batch = p.batch;
  g.win_rows = p.window_rows;
  g.win_cols = p.window_cols;
  if (direction == SNN_HIP_FORWARD) {
    g.p_rows = p.out_rows;  g.p_cols = p.out_cols;
    g.src_rows = p.in_rows; g.src_cols = p.in_cols;
    g.src_ch = p.channels;
    g.step_rows = p.stride_rows; g.step_cols = p.stride_cols;
    g.off_rows = -p.pad_rows;    g.off_cols = -p.pad_cols;
    g.tap_sign = 1;
    g.div_rows = g.div_cols = 1;
    g.n_total = p.features;
  } else {
    g.p_rows = p.in_rows;    g.p_cols = p.in_cols;
    g.src_rows = p.out_rows; g.src_cols = p.out_cols;
    g.src_ch = p.features;
    g.step_rows = g.step_cols = 1;
    g.off_rows = p.pad_rows; g.off_cols = p.pad_cols;
    g.tap_sign = -1;
    g.div_rows = p.stride_rows; g.div_cols = p.stride_cols;
    g.n_total = p.channels;
  }
  g.m_total = g.batch * g.p_rows * g.p_cols;
  g.k_total = g.win_rows * g.win_cols * g.src_ch;
  g.z_src = g.z_wgt = g.z_dst = 0;

  const size_t src_elems = static_cast<size_t>(g.batch) * g.src_rows *
                           g.src_cols * g.src_ch;
  const size_t wgt_elems = static_cast<size_t>(p.window_rows) * p.window_cols *
                           p.channels * p.features;
  if (direction == SNN_HIP_FORWARD && conv2d_stem_supports(p) &&
      (reinterpret_cast<uintptr_t>(output) & 15u) == 0 &&
      SNN_TUNING_ENV("SNN_HIP_STEM_OFF") == nullptr) {
    // three channels, 7x7 stride 2, 64 features: the kernel built for it
    return launch_conv2d_stem_f32(input, filter, output, p, stream);
  }
  if (direction == SNN_HIP_FORWARD && g.src_ch % 4 != 0) {
    launch_scalar_gather_forward(input, filter, output, g, src_elems,
                                 wgt_elems, stream);
  } else if (direction == SNN_HIP_FORWARD) {
    launch_auto<false, false>(input, filter, output, g, src_elems, wgt_elems,
                              stream, epilogue);
  } else if (g.div_rows != 1 || g.div_cols != 1) {
    launch_auto<true, true>(input, filter, output, g, src_elems, wgt_elems,
                            stream, epilogue);
  } else {
    launch_auto<true, false>(input, filter, output, g, src_elems, wgt_elems,
                             stream, epilogue);
  }
  SNN_HIP_CHECK_LAUNCH();
  return SNN_HIP_OK;
}

}  // namespace snn
