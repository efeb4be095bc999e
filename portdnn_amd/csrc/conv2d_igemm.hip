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
};

template <int BM, int BN, int WM, int WN, bool B_K_INNER, bool STRIDED>
__global__ void __launch_bounds__(kThreads)
    conv_igemm_kernel(const float* __restrict__ src,
                      const float* __restrict__ wgt, float* __restrict__ dst,
                      Gather g, unsigned n_tiles_n, unsigned n_blocks) {
  static_assert(WM * WN == 4, "four waves per work-group");
  constexpr int WTM = BM / WM, WTN = BN / WN;  // wave tile
  constexpr int TM = WTM / 32, TN = WTN / 32;  // MFMA blocks per wave
  static_assert(TM >= 1 && TN >= 1, "wave tile must hold a 32x32 block");
  constexpr int A_FLOATS = k_inner_floats(BM);
  constexpr int B_FLOATS =
      B_K_INNER ? k_inner_floats(BN) : row_inner_floats(BN);
  constexpr int STAGE_FLOATS = A_FLOATS + B_FLOATS;
  extern __shared__ __align__(16) float lds[];  // two stages of [A tile | B tile]

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wave_m = wave / WN, wave_n = wave % WN;

  const unsigned tile = xcd_remap(blockIdx.x, n_blocks);
  const int m0 = static_cast<int>(tile / n_tiles_n) * BM;
  const int n0 = static_cast<int>(tile % n_tiles_n) * BN;

  // ---- A gather bookkeeping: this lane copies chunk column `a_cc` (4 floats
  // at k offset 4 * a_cc) of rows a_r0 + 32 * i.
  constexpr int A_ROWS_PER_THREAD = BM / 32;
  const int a_cc = tid & 7;
  const int a_r0 = tid >> 3;
  int a_base[A_ROWS_PER_THREAD];  // element offset of (n, iy0, ix0, 0)
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
      a_base[i] = n * g.src_rows * g.src_cols * g.src_ch;
    } else {
      a_iy0[i] = -(1 << 28);  // never in range
      a_ix0[i] = 0;
      a_base[i] = 0;
    }
  }
  // (tap row, tap col, channel) of this lane's chunk; advanced by BK each step
  int a_c = 4 * a_cc, a_s = 0, a_r = 0;
  while (a_c >= g.src_ch) {
    a_c -= g.src_ch;
    if (++a_s == g.win_cols) { a_s = 0; ++a_r; }
  }

  // ---- B copy bookkeeping
  constexpr int B_VEC_PER_ROW = B_K_INNER ? kBK / 4 : BN / 4;
  constexpr int B_ROWS_PER_PASS = kThreads / B_VEC_PER_ROW;
  constexpr int B_PASSES =
      (B_K_INNER ? BN : kBK) / B_ROWS_PER_PASS;
  const int b_vec = tid % B_VEC_PER_ROW;
  const int b_row0 = tid / B_VEC_PER_ROW;

  float4 a_reg[A_ROWS_PER_THREAD];
  float4 b_reg[B_PASSES];

  auto load_a = [&]() {
    const bool tap_ok = a_r < g.win_rows;
#pragma unroll
    for (int i = 0; i < A_ROWS_PER_THREAD; ++i) {
      int iy = a_iy0[i] + g.tap_sign * a_r;
      int ix = a_ix0[i] + g.tap_sign * a_s;
      bool ok = tap_ok;
      if (STRIDED) {
        ok = ok && iy >= 0 && ix >= 0 && (iy % g.div_rows == 0) &&
             (ix % g.div_cols == 0);
        iy /= g.div_rows;
        ix /= g.div_cols;
      }
      ok = ok && iy >= 0 && iy < g.src_rows && ix >= 0 && ix < g.src_cols;
      float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
      if (ok) {
        v = *reinterpret_cast<const float4*>(
            src + a_base[i] + (iy * g.src_cols + ix) * g.src_ch + a_c);
      }
      a_reg[i] = v;
    }
  };
  auto advance_a = [&]() {
    a_c += kBK;
    while (a_c >= g.src_ch) {
      a_c -= g.src_ch;
      if (++a_s == g.win_cols) { a_s = 0; ++a_r; }
    }
  };
  auto load_b = [&](int k0) {
#pragma unroll
    for (int i = 0; i < B_PASSES; ++i) {
      float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
      if (B_K_INNER) {
        // Wt[q][col]: element (col, q) lives at wgt[(tap * n_total + col) *
        // src_ch + kk] with q = tap * src_ch + kk; rows of the LDS tile are
        // GEMM columns, 4 consecutive q per lane.
        const int col = n0 + b_row0 + B_ROWS_PER_PASS * i;
        const int q = k0 + 4 * b_vec;
        if (col < g.n_total && q < g.k_total) {
          const int tap = q / g.src_ch;
          const int kk = q - tap * g.src_ch;
          v = *reinterpret_cast<const float4*>(
              wgt + (static_cast<size_t>(tap) * g.n_total + col) * g.src_ch +
              kk);
        }
      } else {
        // W[q][col], col contiguous.
        const int q = k0 + b_row0 + B_ROWS_PER_PASS * i;
        const int col = n0 + 4 * b_vec;
        if (q < g.k_total && col < g.n_total) {
          v = *reinterpret_cast<const float4*>(
              wgt + static_cast<size_t>(q) * g.n_total + col);
        }
      }
      b_reg[i] = v;
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

  const int n_chunks = (g.k_total + kBK - 1) / kBK;
  load_a();
  load_b(0);
  advance_a();
  store_tiles(0);
  __syncthreads();
  for (int it = 0; it < n_chunks; ++it) {
    const int stage = it & 1;
    const bool more = it + 1 < n_chunks;
    if (more) {
      load_a();
      load_b((it + 1) * kBK);
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
          dst[static_cast<size_t>(m) * g.n_total + col] = acc[i][j][v];
        }
      }
    }
  }
}

template <int BM, int BN, int WM, int WN, bool B_K_INNER, bool STRIDED>
void launch_tile(const float* src, const float* wgt, float* dst,
                 const Gather& g, hipStream_t stream) {
  const unsigned tiles_m = static_cast<unsigned>(ceil_div(g.m_total, BM));
  const unsigned tiles_n = static_cast<unsigned>(ceil_div(g.n_total, BN));
  const unsigned n_blocks = tiles_m * tiles_n;
  constexpr size_t kLdsBytes =
      2 * sizeof(float) *
      (k_inner_floats(BM) +
       (B_K_INNER ? k_inner_floats(BN) : row_inner_floats(BN)));
  auto kernel = conv_igemm_kernel<BM, BN, WM, WN, B_K_INNER, STRIDED>;
  // More than the 64 KiB default needs an explicit opt-in (160 KiB per CU).
  static const hipError_t attr = hipFuncSetAttribute(
      reinterpret_cast<const void*>(kernel),
      hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes);
  (void)attr;
  hipLaunchKernelGGL(kernel, dim3(n_blocks), dim3(kThreads), kLdsBytes, stream,
                     src, wgt, dst, g, tiles_n, n_blocks);
}

}  // namespace

bool conv2d_igemm_supports(int direction, const snn_hip_conv2d_params& p) {
  if (direction == SNN_HIP_FORWARD)
    return p.channels % 4 == 0 && p.features % 4 == 0;
  if (direction == SNN_HIP_INPUT_BACKPROP)
    return p.features % 4 == 0;
  return false;
}

int launch_conv2d_igemm_f32(int direction, const float* input,
                            const float* filter, float* output,
                            const snn_hip_conv2d_params& p,
                            hipStream_t stream) {
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

  if (direction == SNN_HIP_FORWARD) {
    if (g.n_total > 64)
      launch_tile<128, 128, 2, 2, false, false>(input, filter, output, g, stream);
    else
      launch_tile<128, 64, 4, 1, false, false>(input, filter, output, g, stream);
  } else {
    const bool strided = g.div_rows != 1 || g.div_cols != 1;
    if (strided) {
      launch_tile<128, 64, 4, 1, true, true>(input, filter, output, g, stream);
    } else if (g.n_total > 64) {
      launch_tile<128, 128, 2, 2, true, false>(input, filter, output, g, stream);
    } else {
      launch_tile<128, 64, 4, 1, true, false>(input, filter, output, g, stream);
    }
  }
  SNN_HIP_CHECK_LAUNCH();
  return SNN_HIP_OK;
}

}  // namespace snn
