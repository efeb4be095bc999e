// Half-precision forward convolution as an implicit GEMM on MFMA (gfx950):
// binary16 operands, fp32 accumulation, binary16 result.
//
// Same structure as the fp32 fast path in conv2d_igemm.hip (gathered A tile,
// wave-uniform tap bookkeeping, per-row tap-validity masks, buffer addressing,
// two LDS stages), with the reduction chunk at 64 halves (128 bytes per tile
// row, as in the fp32 kernel) and the contraction on
// v_mfma_f32_32x32x16_f16: lane l supplies A[row = l % 32][k = 8 * (l / 32)
// .. + 7] and the matching B values, i.e. exactly one ds_read_b128 per
// operand per instruction when both tiles keep the reduction index
// contiguous.  The HWCF filter has the feature index contiguous instead, so
// the launcher first rewrites it as [tap][K][C] (a few microseconds for a
// filter of at most a few MB) into the caller's workspace when one is given,
// otherwise into a stream-ordered temporary.
//
// portDNN's half build accumulates in half (e.g. `DataType out_val{0}` with
// T = cl::sycl::half in src/conv2d/direct/kernels_nhwc.h:92); accumulating in
// fp32 is more accurate and stays inside the 1e-2 relative bar against it.
#include <cstdlib>

#include "gemm_tile.h"
#include "snn_kernels.h"

namespace snn {
namespace {

using gemm::float16v;
using gemm::kPad;
using gemm::kThreads;
using gemm::xcd_remap;

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef unsigned int uint4v __attribute__((ext_vector_type(4)));
constexpr int kBKh = 64;             // halves per reduction chunk
constexpr int kRowH = kBKh + 8;      // halves per LDS tile row (16-byte pad)
constexpr unsigned kOob = 0x7FFFFFF0u;
constexpr size_t kMaxBufferBytes = 0x7FFFFFF0u;

struct GatherH {
  int p_rows, p_cols;      // output pixel grid
  int src_rows, src_cols;  // input spatial size
  int src_ch;              // input channels (contiguous)
  int win_rows, win_cols;
  int step_rows, step_cols;
  int off_rows, off_cols;
  int m_total, n_total;
};

__device__ inline __amdgpu_buffer_rsrc_t make_rsrc(const void* p,
                                                   unsigned bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, bytes,
                                           0x00020000);
}

// wt[tap][k][c] = w[tap][c][k]
__global__ void __launch_bounds__(256)
    repack_filter_kernel(const _Float16* __restrict__ w,
                         _Float16* __restrict__ wt, int channels,
                         int features, int n_total) {
  const int idx = blockIdx.x * 256 + threadIdx.x;
  if (idx >= n_total) return;
  const int c = idx % channels;
  const int t = idx / channels;
  const int k = t % features;
  const int tap = t / features;
  wt[idx] = w[(static_cast<size_t>(tap) * channels + c) * features + k];
}

template <int BM, int BN, int WM, int WN>
__global__ void __launch_bounds__(kThreads)
    conv_igemm_f16_kernel(const _Float16* __restrict__ src,
                          const _Float16* __restrict__ wgt_t,
                          _Float16* __restrict__ dst, GatherH g,
                          unsigned src_bytes, unsigned wgt_bytes,
                          unsigned dst_bytes, unsigned n_tiles_n,
                          unsigned n_tiles) {
  static_assert(WM * WN == 4, "four waves per work-group");
  constexpr int WTM = BM / WM, WTN = BN / WN;
  constexpr int TM = WTM / 32, TN = WTN / 32;
  constexpr int A_HALVES = BM * kRowH;
  constexpr int STAGE_HALVES = (BM + BN) * kRowH;
  extern __shared__ __align__(16) _Float16 lds_h[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wave_m = wave / WN, wave_n = wave % WN;
  const unsigned tile = xcd_remap(blockIdx.x, n_tiles);
  const int m0 = static_cast<int>(tile / n_tiles_n) * BM;
  const int n0 = static_cast<int>(tile % n_tiles_n) * BN;
  const int chunks_per_tap = g.src_ch / kBKh;
  const int n_chunks = g.win_rows * g.win_cols * chunks_per_tap;

  const __amdgpu_buffer_rsrc_t src_rsrc = make_rsrc(src, src_bytes);
  const __amdgpu_buffer_rsrc_t wgt_rsrc = make_rsrc(wgt_t, wgt_bytes);

  constexpr int A_PASSES = BM / 32;
  constexpr int B_PASSES = BN / 32;
  const int cc = tid & 7;   // 16-byte column of the 128-byte tile row
  const int r0 = tid >> 3;  // tile row of pass 0
  unsigned a_voff[A_PASSES];
  unsigned a_inval[A_PASSES];
#pragma unroll
  for (int i = 0; i < A_PASSES; ++i) {
    const int m = m0 + r0 + 32 * i;
    unsigned inval = 0xFFFFFFFFu;
    int off = 0;
    if (m < g.m_total) {
      const int px = m % g.p_cols;
      const int t = m / g.p_cols;
      const int py = t % g.p_rows;
      const int n = t / g.p_rows;
      const int iy0 = py * g.step_rows + g.off_rows;
      const int ix0 = px * g.step_cols + g.off_cols;
      off = ((n * g.src_rows + iy0) * g.src_cols + ix0) * g.src_ch + 8 * cc;
      unsigned col_bad = 0;
      for (int c = 0; c < g.win_cols; ++c) {
        const unsigned ix = static_cast<unsigned>(ix0 + c);
        col_bad |= (ix < static_cast<unsigned>(g.src_cols) ? 0u : 1u) << c;
      }
      const unsigned all_cols = (1u << g.win_cols) - 1u;
      inval = 0;
      int shift = 0;
      for (int r = 0; r < g.win_rows; ++r, shift += g.win_cols) {
        const unsigned iy = static_cast<unsigned>(iy0 + r);
        inval |= (iy < static_cast<unsigned>(g.src_rows) ? col_bad : all_cols)
                 << shift;
      }
    }
    a_voff[i] = static_cast<unsigned>(off) * 2u;
    a_inval[i] = inval;
  }
  unsigned b_voff[B_PASSES];
#pragma unroll
  for (int i = 0; i < B_PASSES; ++i) {
    const int col = n0 + r0 + 32 * i;
    b_voff[i] = col < g.n_total
                    ? static_cast<unsigned>(col * g.src_ch + 8 * cc) * 2u
                    : kOob;
  }
  const unsigned b_tap_stride =
      static_cast<unsigned>(g.n_total * g.src_ch) * 2u;

  int tap = 0, c0 = 0, tap_r = 0, tap_c = 0, chunk = 0;
  uint4v a_reg[A_PASSES], b_reg[B_PASSES];
  auto load_global = [&]() {
    if (chunk >= n_chunks) return;
    const unsigned a_soff = static_cast<unsigned>(
        ((tap_r * g.src_cols + tap_c) * g.src_ch + c0) * 2);
#pragma unroll
    for (int i = 0; i < A_PASSES; ++i) {
      const unsigned bad = __builtin_amdgcn_ubfe(a_inval[i], tap, 1);
      a_reg[i] = __builtin_amdgcn_raw_buffer_load_b128(
          src_rsrc, (bad << 31) | (a_voff[i] + a_soff), 0, 0);
    }
    const unsigned b_soff = static_cast<unsigned>(tap) * b_tap_stride +
                            static_cast<unsigned>(c0) * 2u;
#pragma unroll
    for (int i = 0; i < B_PASSES; ++i) {
      b_reg[i] = __builtin_amdgcn_raw_buffer_load_b128(wgt_rsrc, b_voff[i],
                                                       b_soff, 0);
    }
    ++chunk;
    c0 += kBKh;
    if (c0 == g.src_ch) {
      c0 = 0;
      ++tap;
      if (++tap_c == g.win_cols) { tap_c = 0; ++tap_r; }
    }
  };
  _Float16* const a_store = lds_h + r0 * kRowH + 8 * cc;
  _Float16* const b_store = lds_h + A_HALVES + r0 * kRowH + 8 * cc;
  auto store_tiles = [&](int stage) {
#pragma unroll
    for (int i = 0; i < A_PASSES; ++i)
      *reinterpret_cast<uint4v*>(a_store + stage * STAGE_HALVES +
                                 32 * i * kRowH) = a_reg[i];
#pragma unroll
    for (int i = 0; i < B_PASSES; ++i)
      *reinterpret_cast<uint4v*>(b_store + stage * STAGE_HALVES +
                                 32 * i * kRowH) = b_reg[i];
  };

  float16v acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  const int l32 = lane & 31;
  const int k_half = 8 * (lane >> 5);
  auto compute = [&](int stage) {
    const _Float16* a_tile = lds_h + stage * STAGE_HALVES;
    const _Float16* b_tile = a_tile + A_HALVES;
    half8 a[kBKh / 16][TM], b[kBKh / 16][TN];
#pragma unroll
    for (int s = 0; s < kBKh / 16; ++s) {
#pragma unroll
      for (int i = 0; i < TM; ++i)
        a[s][i] = *reinterpret_cast<const half8*>(
            a_tile + (wave_m * WTM + 32 * i + l32) * kRowH + 16 * s + k_half);
#pragma unroll
      for (int j = 0; j < TN; ++j)
        b[s][j] = *reinterpret_cast<const half8*>(
            b_tile + (wave_n * WTN + 32 * j + l32) * kRowH + 16 * s + k_half);
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int s = 0; s < kBKh / 16; ++s)
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(
              a[s][i], b[s][j], acc[i][j], 0, 0, 0);
  };

  load_global();
  store_tiles(0);
  __syncthreads();
  for (int done = 0;; done += 2) {
    load_global();
    compute(0);
    if (done + 1 >= n_chunks) break;
    store_tiles(1);
    __syncthreads();
    load_global();
    compute(1);
    if (done + 2 >= n_chunks) break;
    store_tiles(0);
    __syncthreads();
  }

  const __amdgpu_buffer_rsrc_t dst_rsrc = make_rsrc(dst, dst_bytes);
  const unsigned row_bytes = static_cast<unsigned>(g.n_total) * 2u;
#pragma unroll
  for (int i = 0; i < TM; ++i) {
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int col = n0 + wave_n * WTN + 32 * j + l32;
      const int m_base = m0 + wave_m * WTM + 32 * i + 4 * (lane >> 5);
      const unsigned voff =
          (col < g.n_total && m_base < g.m_total)
              ? static_cast<unsigned>(m_base) * row_bytes +
                    static_cast<unsigned>(col) * 2u
              : kOob;
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const unsigned off =
            voff + static_cast<unsigned>(8 * (v >> 2) + (v & 3)) * row_bytes;
        const _Float16 h = static_cast<_Float16>(acc[i][j][v]);
        __builtin_amdgcn_raw_buffer_store_b16(
            __builtin_bit_cast(unsigned short, h), dst_rsrc, off, 0, 0);
      }
    }
  }
}

template <int BM, int BN, int WM, int WN>
void launch_f16_tile(const _Float16* src, const _Float16* wgt_t, _Float16* dst,
                     const GatherH& g, size_t src_elems, size_t wgt_elems,
                     hipStream_t stream) {
  const unsigned tiles_m = static_cast<unsigned>(ceil_div(g.m_total, BM));
  const unsigned tiles_n = static_cast<unsigned>(ceil_div(g.n_total, BN));
  const unsigned n_tiles = tiles_m * tiles_n;
  constexpr size_t kLdsBytes = 2 * sizeof(_Float16) * (BM + BN) * kRowH;
  auto kernel = conv_igemm_f16_kernel<BM, BN, WM, WN>;
  static const hipError_t attr = hipFuncSetAttribute(
      reinterpret_cast<const void*>(kernel),
      hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes);
  (void)attr;
  KernelTimer timer(stream);
  hipLaunchKernelGGL(
      kernel, dim3(n_tiles), dim3(kThreads), kLdsBytes, stream, src, wgt_t, dst,
      g, static_cast<unsigned>(src_elems * 2),
      static_cast<unsigned>(wgt_elems * 2),
      static_cast<unsigned>(static_cast<size_t>(g.m_total) * g.n_total * 2),
      tiles_n, n_tiles);
}

}  // namespace

bool conv2d_igemm_f16_supports(const snn_hip_conv2d_params& p) {
  const size_t x = static_cast<size_t>(p.batch) * p.in_rows * p.in_cols *
                   p.channels;
  const size_t y = static_cast<size_t>(p.batch) * p.out_rows * p.out_cols *
                   p.features;
  return p.channels % kBKh == 0 && p.window_rows * p.window_cols <= 32 &&
         p.window_cols < 32 &&
         (x > y ? x : y) * 2 <= kMaxBufferBytes;
}

int launch_conv2d_igemm_f16(const _Float16* input, const _Float16* filter,
                            _Float16* output, const snn_hip_conv2d_params& p,
                            _Float16* workspace, size_t workspace_elems,
                            hipStream_t stream) {
  const size_t wgt_elems = static_cast<size_t>(p.window_rows) * p.window_cols *
                           p.channels * p.features;
  // 1x1, stride 1, no padding: a plain row-major GEMM over the pixels
  if (p.window_rows == 1 && p.window_cols == 1 && p.stride_rows == 1 &&
      p.stride_cols == 1 && p.pad_rows == 0 && p.pad_cols == 0 &&
      p.out_rows == p.in_rows && p.out_cols == p.in_cols &&
      ((reinterpret_cast<uintptr_t>(input) |
        reinterpret_cast<uintptr_t>(filter) |
        reinterpret_cast<uintptr_t>(output)) & 15u) == 0) {
    const size_t pixels = static_cast<size_t>(p.batch) * p.in_rows * p.in_cols;
    if (pixels <= static_cast<size_t>(INT_MAX) &&
        gemm_rows_f16_supports(static_cast<int>(pixels), p.channels,
                               p.features))
      return launch_gemm_rows_f16(input, filter, output,
                                  static_cast<int>(pixels), p.channels,
                                  p.features, stream);
  }
  _Float16* wgt_t = workspace;
  bool temporary = false;
  if (workspace == nullptr || workspace_elems < wgt_elems ||
      (reinterpret_cast<uintptr_t>(workspace) & 15u) != 0) {
    void* ptr = nullptr;
    if (temp_malloc_async(&ptr, wgt_elems * sizeof(_Float16), stream) != hipSuccess)
      return SNN_HIP_ALLOCATION_PROBLEM;
    wgt_t = static_cast<_Float16*>(ptr);
    temporary = true;
  }
  static const bool no_rowtile = SNN_TUNING_ENV("SNN_HIP_F16_IGEMM") != nullptr;
  if (!no_rowtile && conv2d_rowtile_f16_supports(p)) {
    const int status =
        launch_conv2d_rowtile_f16(input, filter, output, p, wgt_t, stream);
    if (temporary) temp_free_async(wgt_t, stream);
    return status;
  }
  hipLaunchKernelGGL(repack_filter_kernel,
                     dim3(static_cast<unsigned>(ceil_div(wgt_elems, size_t{256}))),
                     dim3(256), 0, stream, filter, wgt_t, p.channels,
                     p.features, static_cast<int>(wgt_elems));
  GatherH g;
  g.p_rows = p.out_rows; g.p_cols = p.out_cols;
  g.src_rows = p.in_rows; g.src_cols = p.in_cols;
  g.src_ch = p.channels;
  g.win_rows = p.window_rows; g.win_cols = p.window_cols;
  g.step_rows = p.stride_rows; g.step_cols = p.stride_cols;
  g.off_rows = -p.pad_rows; g.off_cols = -p.pad_cols;
  g.m_total = p.batch * p.out_rows * p.out_cols;
  g.n_total = p.features;
  const size_t src_elems =
      static_cast<size_t>(p.batch) * p.in_rows * p.in_cols * p.channels;
  const long big = static_cast<long>(ceil_div(g.m_total, 128)) *
                   ceil_div(g.n_total, 128);
  if (g.n_total > 64 && big >= 512)
    launch_f16_tile<128, 128, 2, 2>(input, wgt_t, output, g, src_elems,
                                    wgt_elems, stream);
  else
    launch_f16_tile<64, 64, 2, 2>(input, wgt_t, output, g, src_elems,
                                  wgt_elems, stream);
  const hipError_t launch_err = hipGetLastError();
  if (temporary) temp_free_async(wgt_t, stream);
  if (launch_err != hipSuccess)
    return report_hip_error(launch_err, "conv_igemm_f16_kernel");
  return SNN_HIP_OK;
}

// The input gradient of a stride-1 convolution as a forward convolution of
// dY: channels and features trade places, padding becomes window - 1 - pad.
static bool as_forward_of_dy(const snn_hip_conv2d_params& p,
                             snn_hip_conv2d_params* q) {
  if (p.stride_rows != 1 || p.stride_cols != 1) return false;
  if (p.pad_rows > p.window_rows - 1 || p.pad_cols > p.window_cols - 1)
    return false;
  *q = p;
  q->channels = p.features;
  q->features = p.channels;
  q->in_rows = p.out_rows;
  q->in_cols = p.out_cols;
  q->out_rows = p.in_rows;
  q->out_cols = p.in_cols;
  q->pad_rows = p.window_rows - 1 - p.pad_rows;
  q->pad_cols = p.window_cols - 1 - p.pad_cols;
  return true;
}

// Halves of caller workspace the forward / input-gradient launchers below put
// to use (the re-laid-out filter); 0 for the shapes that need none.
size_t conv2d_f16_filter_pack_halves(int direction,
                                     const snn_hip_conv2d_params& p) {
  const size_t wgt_elems = static_cast<size_t>(p.window_rows) * p.window_cols *
                           p.channels * p.features;
  if (direction == SNN_HIP_FORWARD) {
    if (!conv2d_igemm_f16_supports(p)) return 0;
    const size_t pixels = static_cast<size_t>(p.batch) * p.in_rows * p.in_cols;
    if (p.window_rows == 1 && p.window_cols == 1 && p.stride_rows == 1 &&
        p.stride_cols == 1 && p.pad_rows == 0 && p.pad_cols == 0 &&
        p.out_rows == p.in_rows && p.out_cols == p.in_cols &&
        pixels <= static_cast<size_t>(INT_MAX) &&
        gemm_rows_f16_supports(static_cast<int>(pixels), p.channels,
                               p.features))
      return 0;
    return wgt_elems;
  }
  if (direction == SNN_HIP_INPUT_BACKPROP) {
    snn_hip_conv2d_params q;
    if (!as_forward_of_dy(p, &q)) return 0;
    return conv2d_rowtile_f16_supports(q) ? wgt_elems : 0;
  }
  return 0;
}

bool conv2d_input_backprop_f16_supports(const snn_hip_conv2d_params& p) {
  snn_hip_conv2d_params q;
  if (!as_forward_of_dy(p, &q)) return false;
  if (conv2d_rowtile_f16_supports(q)) return true;
  // 1x1: W[c][k] already is the gradient's filter with the reduction index
  // (k) contiguous, the layout the implicit-GEMM kernel wants
  return p.window_rows == 1 && p.window_cols == 1 &&
         conv2d_igemm_f16_supports(q);
}

int launch_conv2d_input_backprop_f16(const _Float16* dy,
                                     const _Float16* filter, _Float16* dx,
                                     const snn_hip_conv2d_params& p,
                                     _Float16* workspace,
                                     size_t workspace_elems,
                                     hipStream_t stream) {
  snn_hip_conv2d_params q;
  if (!as_forward_of_dy(p, &q)) return SNN_HIP_INVALID_ALGORITHM;
  const size_t wgt_elems = static_cast<size_t>(p.window_rows) * p.window_cols *
                           p.channels * p.features;
  if (conv2d_rowtile_f16_supports(q)) {
    _Float16* packed = workspace;
    bool temporary = false;
    if (workspace == nullptr || workspace_elems < wgt_elems ||
        (reinterpret_cast<uintptr_t>(workspace) & 15u) != 0) {
      void* ptr = nullptr;
      if (temp_malloc_async(&ptr, wgt_elems * sizeof(_Float16), stream) !=
          hipSuccess)
        return SNN_HIP_ALLOCATION_PROBLEM;
      packed = static_cast<_Float16*>(ptr);
      temporary = true;
    }
    const int status =
        launch_conv2d_rowtile_f16(dy, filter, dx, q, packed, stream, true);
    if (temporary) temp_free_async(packed, stream);
    return status;
  }
  if (p.window_rows != 1 || p.window_cols != 1 || !conv2d_igemm_f16_supports(q))
    return SNN_HIP_INVALID_ALGORITHM;
  GatherH g;
  g.p_rows = q.out_rows; g.p_cols = q.out_cols;
  g.src_rows = q.in_rows; g.src_cols = q.in_cols;
  g.src_ch = q.channels;
  g.win_rows = 1; g.win_cols = 1;
  g.step_rows = 1; g.step_cols = 1;
  g.off_rows = -q.pad_rows; g.off_cols = -q.pad_cols;
  g.m_total = q.batch * q.out_rows * q.out_cols;
  g.n_total = q.features;
  const size_t src_elems =
      static_cast<size_t>(q.batch) * q.in_rows * q.in_cols * q.channels;
  const long big = static_cast<long>(ceil_div(g.m_total, 128)) *
                   ceil_div(g.n_total, 128);
  if (g.n_total > 64 && big >= 512)
    launch_f16_tile<128, 128, 2, 2>(dy, filter, dx, g, src_elems, wgt_elems,
                                    stream);
  else
    launch_f16_tile<64, 64, 2, 2>(dy, filter, dx, g, src_elems, wgt_elems,
                                  stream);
  const hipError_t launch_err = hipGetLastError();
  if (launch_err != hipSuccess)
    return report_hip_error(launch_err, "conv_igemm_f16_kernel");
  return SNN_HIP_OK;
}

}  // namespace snn
