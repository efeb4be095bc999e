// Forward convolution of an image with three channels: 7x7 window, stride 2,
// 64 features, fp32 NHWC x HWCF -- the ResNet stem (the forward case of
// include/portdnn/conv2d/launch.h:59-118 that the reference runs on its Direct /
// Tiled kernels, src/conv2d/direct/kernels.h, src/conv2d/tiled/kernels.h).
// As an implicit GEMM this layer has a reduction of 7 * 7 * 3 = 147 with the
// three channels innermost, which neither 16-byte gathers nor whole chunks of
// 32 fit; the general kernel locates and loads every reduction index on its
// own.  Here the structure of the layer is used instead:
//
//   * a work-group owns a band of consecutive output rows of one image and
//     keeps every input row the band touches in LDS, each loaded once with
//     `buffer_load_dword ... lds` (no registers; rows and columns of the
//     padding arrive as zeros through the buffer range check).  An input row
//     is stored from its left padding on, so the 7 * 3 = 21 reduction values
//     of one filter row are 21 consecutive floats at 6 * ox for output column
//     ox, and 16 neighbouring output pixels read them without bank conflicts
//     (stride 6 words);
//   * the filter sits in registers, a quarter (16 features) per wave: 37 matrix
//     instructions of 4 reduction indices (148, the last one a zero weight
//     whose operand comes from a word of LDS that holds zero);
//   * a wave multiplies blocks of 16 output pixels against its 16 features,
//     v_mfma_f32_16x16x4_f32 with features as rows, so a lane ends with four
//     consecutive features of its pixel (16-byte stores).
//
// Reduction order inside an output: k = 4 t + q for instruction t and lane
// quarter q, summed by the matrix unit over q and accumulated over t in order.
#include <algorithm>

#include "snn_kernels.h"

namespace snn {
namespace {

typedef float float4v __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) void* lds_ptr;

constexpr int kWaves = 8;
constexpr int kWin = 7, kCh = 3, kStride = 2, kFeatures = 64;
constexpr int kRowK = kWin * kCh;                 // 21 reduction values per filter row
constexpr int kK = kWin * kRowK;                  // 147
constexpr int kSteps = (kK + 3) / 4;              // 37 matrix instructions per block
constexpr unsigned kOobOffset = 0x7FFFFFF0u;
constexpr size_t kMaxBufferBytes = 0x7FFFFFF0u;
constexpr size_t kMaxLdsBytes = 150 * 1024;
constexpr int kStoreAux = 2;  // the output is written once: stream it (slc)

__device__ inline __amdgpu_buffer_rsrc_t make_rsrc(const void* p,
                                                   size_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0,
                                           static_cast<unsigned>(bytes),
                                           0x00020000);
}

constexpr int vmcnt_imm(int n) {
  return 0x0F70 | (n & 15) | ((n >> 4) << 14);
}

struct StemGeom {
  int batch, in_rows, in_cols, out_rows, out_cols, pad_rows, pad_cols;
  int band;        // output rows per work-group (even)
  int n_bands;     // bands per image
  int row_floats;  // LDS floats per input row (a multiple of 64)
  int lds_rows;    // 2 * band + 5
  int loads_per_row;   // row_floats / 64
};

constexpr int kNpb = 7;              // 16-pixel blocks of an output row
constexpr int kUnits = kNpb;         // (output row, pixel block) pairs per wave and step
constexpr int kRowsPerStep = 2;      // output rows per step
constexpr int kNewRows = kStride * kRowsPerStep;  // input rows a step adds
constexpr int kGroup = 4;            // matrix instructions per operand fetch
// LDS floats per input row, fixed so that operand addresses are immediates:
// 11 x 64 floats hold the 224 + 6 columns a 112-pixel output row reads.
constexpr int kRowFloats = 704;
// Fewest output rows (over the batch) the kernel is used for.
constexpr long kMinOutputRows = 224;

// Reduction index k = 4 t + q sits k / 21 rows down and k % 21 floats along.
// For most t the four lane quarters stay in one filter row, so the offset is
// a constant plus q and the constant goes into the instruction; where a row
// ends inside the group (and in the last group, which has one index past
// the reduction) a lane needs an offset of its own.
constexpr bool group_straddles(int t) {
  return (4 * t) / kRowK != (4 * t + 3) / kRowK || 4 * t + 3 >= kK;
}
constexpr int group_offset(int t) {
  return ((4 * t) / kRowK) * kRowFloats + (4 * t) % kRowK;
}
constexpr int count_straddles() {
  int n = 0;
  for (int t = 0; t < kSteps; ++t) n += group_straddles(t) ? 1 : 0;
  return n;
}
constexpr int straddle_index(int t) {
  int n = 0;
  for (int u = 0; u < t; ++u) n += group_straddles(u) ? 1 : 0;
  return n;
}
constexpr int kStraddles = count_straddles();

// Input rows of the band go to LDS row 0 ...; LDS column i of a row holds the
// input float i - 3 * pad_cols of that image row.
//
// A step is two output rows = 2 x 7 pixel blocks x 4 feature blocks = 56
// blocks of 16 x 16 outputs, seven per wave: wave w takes blocks w, w + 8, ...,
// in (row, pixel block, feature block) order, which gives it the feature block
// w % 4 every time -- it keeps that quarter of the filter (37 registers) -- and
// the four SIMDs the same work (with one output row per step and one pixel
// block per wave the eighth wave idled).
// TY: the output's element type (fp32, or binary16 rounded on the store for
// the binary16 launch, whose 64-feature tensor is the large one).
template <typename TY>
__global__ void __launch_bounds__(64 * kWaves)
    __attribute__((amdgpu_waves_per_eu(2, 2)))
    conv_stem_7x7s2_kernel(const float* __restrict__ x,
                           const float* __restrict__ w, TY* __restrict__ y,
                           StemGeom g) {
  extern __shared__ __align__(16) float lds[];
  // one word past the rows that always holds zero
  const int zero_word = g.lds_rows * kRowFloats;
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int q = lane >> 4;
  const int px = lane & 15;
  const int fb = wave & 3;
  const int n = blockIdx.x / g.n_bands;
  const int band = blockIdx.x % g.n_bands;
  const int oy0 = band * g.band;
  const int n_rows = min(g.band, g.out_rows - oy0);
  const int n_steps = (n_rows + kRowsPerStep - 1) / kRowsPerStep;
  const int y_first = kStride * oy0 - g.pad_rows;

  const __amdgpu_buffer_rsrc_t x_rsrc = make_rsrc(
      x, static_cast<size_t>(g.batch) * g.in_rows * g.in_cols * kCh * 4);
  const __amdgpu_buffer_rsrc_t y_rsrc = make_rsrc(
      y, static_cast<size_t>(g.batch) * g.out_rows * g.out_cols * kFeatures *
             sizeof(TY));

  if (threadIdx.x == 0) lds[zero_word] = 0.f;

  // Load instruction `i` of LDS row `row`: 64 consecutive floats.  A row or a
  // column outside the image is out of the buffer's range: zeros.
  const int row_bytes_in = g.in_cols * kCh * 4;
  auto issue_row_piece = [&](int row, int i, bool live) {
    const int yy = y_first + row;
    const int f = i * 64 + lane - kCh * g.pad_cols;  // float index in the image row
    const bool ok = live &&
                    static_cast<unsigned>(yy) < static_cast<unsigned>(g.in_rows) &&
                    static_cast<unsigned>(f) <
                        static_cast<unsigned>(g.in_cols * kCh);
    const unsigned off =
        ok ? static_cast<unsigned>((n * g.in_rows + yy)) *
                     static_cast<unsigned>(row_bytes_in) +
                 static_cast<unsigned>(f) * 4u
           : kOobOffset;
    __builtin_amdgcn_raw_ptr_buffer_load_lds(
        x_rsrc, (lds_ptr)(lds + row * kRowFloats + i * 64), 4, off, 0, 0, 0);
  };
  // this wave's quarter of the filter, in matrix-operand order: k = 4 t + q,
  // feature 16 fb + px
  float wreg[kSteps];
#pragma unroll
  for (int t = 0; t < kSteps; ++t) {
    const int k = 4 * t + q;
    wreg[t] = k < kK ? w[k * kFeatures + 16 * fb + px] : 0.f;
  }
  // the lanes' own offsets for the groups that straddle a filter row, relative
  // to a block's base (which already includes q); the index past the
  // reduction reads the zero word instead: its weight is zero, but zero times a
  // stray infinity would not be
  int kspec[kStraddles];
#pragma unroll
  for (int t = 0; t < kSteps; ++t) {
    if (group_straddles(t)) {
      const int k = 4 * t + q;
      kspec[straddle_index(t)] =
          k < kK ? (k / kRowK) * kRowFloats + k % kRowK - q : 0;
    }
  }
  const bool last_is_pad = 4 * (kSteps - 1) + q >= kK;
  // this wave's blocks of a step: output row u / 28 of the step, pixel block
  // (u % 28) / 4 for u = wave + 8 i
  int unit_row[kUnits], unit_pb[kUnits];
#pragma unroll
  for (int i = 0; i < kUnits; ++i) {
    const int u = wave + kWaves * i;
    unit_row[i] = u / (4 * kNpb);
    unit_pb[i] = (u % (4 * kNpb)) >> 2;
  }

  // ---- start: the rows of the first two steps are waited for; every other
  // row of the band is issued behind them and has two steps to arrive.  The
  // band's rows all have a place of their own in LDS, so nothing is ever
  // overwritten and two barriers serve the whole band.
  constexpr int kFirstRows = kWin - kStride + 2 * kNewRows;
  __builtin_amdgcn_sched_barrier(0);
  for (int row = 0; row < kFirstRows && row < g.lds_rows; ++row)
    for (int i = wave; i < g.loads_per_row; i += kWaves)
      issue_row_piece(row, i, true);
  __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
  __syncthreads();
  for (int row = kFirstRows; row < g.lds_rows; ++row)
    for (int i = wave; i < g.loads_per_row; i += kWaves)
      issue_row_piece(row, i, true);

  for (int s = 0; s < n_steps; ++s) {
    if (s == 2) {
      // Vector-memory operations retire in order: once at most the stores of
      // the first two steps are outstanding, every load has landed.
      __builtin_amdgcn_sched_barrier(0);
      __builtin_amdgcn_s_waitcnt(vmcnt_imm(2 * kUnits));
      __builtin_amdgcn_s_barrier();
      __builtin_amdgcn_sched_barrier(0);
    }
    // where each block's windows start in LDS; a block outside the image or
    // the band computes on the first block's data and is not stored
    const float* base[kUnits];
    bool live[kUnits];
#pragma unroll
    for (int i = 0; i < kUnits; ++i) {
      live[i] = kRowsPerStep * s + unit_row[i] < n_rows &&
                16 * unit_pb[i] < g.out_cols;
      const int row0 = live[i] ? kNewRows * s + kStride * unit_row[i]
                               : kNewRows * s;
      const int pb = live[i] ? unit_pb[i] : 0;
      base[i] = lds + row0 * kRowFloats + kStride * kCh * (16 * pb + px) + q;
    }
    float4v acc[kUnits];
#pragma unroll
    for (int i = 0; i < kUnits; ++i) acc[i] = float4v{0.f, 0.f, 0.f, 0.f};
    // operands are fetched one group of matrix instructions ahead; the seven
    // blocks take turns, so consecutive instructions never share an
    // accumulator
    float xv[2][kGroup][kUnits];
    auto fetch = [&](int t0, float (&dst)[kGroup][kUnits]) {
#pragma unroll
      for (int e = 0; e < kGroup; ++e) {
        const int t = t0 + e;
        if (t < kSteps) {
#pragma unroll
          for (int i = 0; i < kUnits; ++i) {
            const float* src = group_straddles(t)
                                   ? base[i] + kspec[straddle_index(t)]
                                   : base[i] + group_offset(t);
            if (t == kSteps - 1) src = last_is_pad ? lds + zero_word : src;
            dst[e][i] = *src;
          }
        }
      }
    };
    fetch(0, xv[0]);
#pragma unroll
    for (int t0 = 0; t0 < kSteps; t0 += kGroup) {
      // (fences: the compiler otherwise sinks each fetch to its use)
      __builtin_amdgcn_sched_barrier(0);
      if (t0 + kGroup < kSteps) fetch(t0 + kGroup, xv[(t0 / kGroup + 1) & 1]);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int e = 0; e < kGroup; ++e) {
        const int t = t0 + e;
        if (t < kSteps) {
#pragma unroll
          for (int i = 0; i < kUnits; ++i)
            acc[i] = __builtin_amdgcn_mfma_f32_16x16x4f32(
                wreg[t], xv[(t0 / kGroup) & 1][e][i], acc[i], 0, 0, 0);
        }
      }
    }
#pragma unroll
    for (int i = 0; i < kUnits; ++i) {
      const int oy = oy0 + kRowsPerStep * s + unit_row[i];
      const int ox = 16 * unit_pb[i] + px;
      const unsigned off =
          (live[i] && ox < g.out_cols)
              ? static_cast<unsigned>(((n * g.out_rows + oy) * g.out_cols + ox) *
                                          kFeatures +
                                      16 * fb + 4 * q) *
                    static_cast<unsigned>(sizeof(TY))
              : kOobOffset;
      if constexpr (sizeof(TY) == 4) {
        __builtin_amdgcn_raw_buffer_store_b128(acc[i], y_rsrc, off, 0,
                                               kStoreAux);
      } else {
        typedef _Float16 half4v __attribute__((ext_vector_type(4)));
        typedef unsigned int uint2v __attribute__((ext_vector_type(2)));
        const float4v r = __builtin_bit_cast(float4v, acc[i]);
        half4v h;
#pragma unroll
        for (int e = 0; e < 4; ++e) h[e] = static_cast<_Float16>(r[e]);
        __builtin_amdgcn_raw_buffer_store_b64(__builtin_bit_cast(uint2v, h),
                                              y_rsrc, off, 0, kStoreAux);
      }
    }
  }
  __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
}

bool make_geom(const snn_hip_conv2d_params& p, StemGeom* g) {
  if (p.channels != kCh || p.features != kFeatures || p.window_rows != kWin ||
      p.window_cols != kWin || p.stride_rows != kStride ||
      p.stride_cols != kStride)
    return false;
  if (p.pad_rows < 0 || p.pad_cols < 0 || p.pad_rows >= kWin ||
      p.pad_cols >= kWin || p.out_cols > 16 * kNpb || p.out_rows < 1)
    return false;
  const size_t in_bytes = static_cast<size_t>(p.batch) * p.in_rows * p.in_cols *
                          kCh * sizeof(float);
  const size_t out_bytes = static_cast<size_t>(p.batch) * p.out_rows *
                           p.out_cols * kFeatures * sizeof(float);
  if (in_bytes > kMaxBufferBytes || out_bytes > kMaxBufferBytes) return false;
  g->batch = p.batch; g->in_rows = p.in_rows; g->in_cols = p.in_cols;
  g->out_rows = p.out_rows; g->out_cols = p.out_cols;
  g->pad_rows = p.pad_rows; g->pad_cols = p.pad_cols;
  // a row holds every column a window of the last output pixel block reads
  const int cols_read = kStride * (16 * ceil_div(p.out_cols, 16) - 1) + kWin;
  if (max(cols_read, p.in_cols + p.pad_cols) * kCh > kRowFloats) return false;
  g->row_floats = kRowFloats;
  g->loads_per_row = g->row_floats / 64;
  // Below two images' worth of rows a band is a single step and the
  // work-group's start-up (filter, first rows) is most of its time: the
  // general kernels are quicker there.
  if (static_cast<long>(p.batch) * p.out_rows < kMinOutputRows) return false;
  // Bands per image: the count whose rounds of work-groups over the CUs,
  // times the steps (plus start-up) of one work-group, come to the least,
  // among those whose rows fit LDS and that give every CU a work-group when
  // the layer has that many steps at all.
  const int n_cus = 256;
  const int max_bands = ceil_div(p.out_rows, kRowsPerStep);
  long best_cost = -1;
  for (int n_bands = 1; n_bands <= max_bands; ++n_bands) {
    // whole steps of two output rows
    const int band =
        ceil_div(ceil_div(p.out_rows, n_bands), kRowsPerStep) * kRowsPerStep;
    const int bands = ceil_div(p.out_rows, band);
    const int lds_rows = kStride * band + kWin - kStride;
    const size_t bytes =
        (static_cast<size_t>(lds_rows + 1) * g->row_floats + 64) * sizeof(float);
    if (bytes > kMaxLdsBytes) continue;
    const size_t groups = static_cast<size_t>(p.batch) * bands;
    const long rounds =
        static_cast<long>(ceil_div(groups, static_cast<size_t>(n_cus)));
    // start-up counted as a step and a half (in half steps)
    const long cost = rounds * (band + 3);
    if (best_cost < 0 || cost < best_cost) {
      best_cost = cost;
      g->band = band;
      g->n_bands = bands;
      g->lds_rows = lds_rows;
    }
  }
  return best_cost >= 0;
}

// ---------------------------------------------------------------------------
// Filter gradient of the same layer:
//   dW[rho][k] = sum over (n, oy, ox) of X[n][2 oy + r - pad][2 ox + s - pad][c] * dY[n][oy][ox][k],
// rho = 21 r + 3 s + c (147 values, ten row blocks of 16, the last 13 rows
// unused).  The work-group and its band of input rows in LDS are the forward
// kernel's.  Matrix instruction: D[rho][k] (16 x 16) += A[rho][4 pixels] *
// B[4 pixels][k]; the A operand of lane l is one LDS float at
// (row 2 (oy - oy0) + rho / 21, column 6 ox + rho % 21), i.e. a per-lane
// constant plus 24 floats per step of four pixels -- an immediate offset; the
// B operand is one float of dY, loaded from global memory a whole output row
// ahead (56 registers).  Wave w: row blocks 5 (w & 1) ... + 4, feature blocks
// 2 ((w >> 1) & 1) ... + 1, output rows of the band of parity w >> 2: 7 loads
// per 10 matrix instructions.  The two parities meet through LDS, the
// work-groups through partial filters that a second kernel sums.
constexpr int kRhoBlocks = 5;   // per wave (ten in all)
constexpr int kMaxTSteps = 28;  // four-pixel steps of an output row
constexpr int kPartFloats = kK * kFeatures;

__global__ void __launch_bounds__(64 * kWaves)
    __attribute__((amdgpu_waves_per_eu(2, 2)))
    conv_stem_filter_backprop_kernel(const float* __restrict__ x,
                                     const float* __restrict__ dy,
                                     float* __restrict__ part, StemGeom g) {
  extern __shared__ __align__(16) float lds[];
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int q = lane >> 4;
  const int l16 = lane & 15;
  const int rh = wave & 1, kp = (wave >> 1) & 1, ph = wave >> 2;
  const int n = blockIdx.x / g.n_bands;
  const int band = blockIdx.x % g.n_bands;
  const int oy0 = band * g.band;
  const int oy_end = min(oy0 + g.band, g.out_rows);
  const int y_first = kStride * oy0 - g.pad_rows;

  const __amdgpu_buffer_rsrc_t x_rsrc = make_rsrc(
      x, static_cast<size_t>(g.batch) * g.in_rows * g.in_cols * kCh * 4);
  const __amdgpu_buffer_rsrc_t dy_rsrc = make_rsrc(
      dy, static_cast<size_t>(g.batch) * g.out_rows * g.out_cols * kFeatures * 4);

  // every input row of the band (rows and columns outside the image: zeros)
  const int row_bytes_in = g.in_cols * kCh * 4;
  for (int row = 0; row < g.lds_rows; ++row)
    for (int i = wave; i < g.loads_per_row; i += kWaves) {
      const int yy = y_first + row;
      const int f = i * 64 + lane - kCh * g.pad_cols;
      const bool ok =
          static_cast<unsigned>(yy) < static_cast<unsigned>(g.in_rows) &&
          static_cast<unsigned>(f) < static_cast<unsigned>(g.in_cols * kCh);
      const unsigned off =
          ok ? static_cast<unsigned>((n * g.in_rows + yy)) *
                       static_cast<unsigned>(row_bytes_in) +
                   static_cast<unsigned>(f) * 4u
             : kOobOffset;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(
          x_rsrc, (lds_ptr)(lds + row * kRowFloats + i * 64), 4, off, 0, 0, 0);
    }

  // A operand: where this lane's rho sits relative to (first LDS row of the
  // output row, pixel 4 t)
  int a_off[kRhoBlocks];
#pragma unroll
  for (int b = 0; b < kRhoBlocks; ++b) {
    const int rho = 16 * (kRhoBlocks * rh + b) + l16;
    a_off[b] = (rho / kRowK) * kRowFloats + 6 * q + rho % kRowK;
  }
  const int n_tsteps = (g.out_cols + 3) >> 2;
  const int n_iter = (g.band + 1) >> 1;  // output rows per parity

  float4v acc[kRhoBlocks][2];
#pragma unroll
  for (int b = 0; b < kRhoBlocks; ++b)
#pragma unroll
    for (int j = 0; j < 2; ++j) acc[b][j] = float4v{0.f, 0.f, 0.f, 0.f};

  // dY of one output row for this lane: pixel 4 t + q, features
  // 16 (2 kp + j) + l16; zeros past the row's end and past the band's.  One
  // per-lane offset per row, the step and the feature block in the scalar
  // offset, so that a row's 56 loads cost no vector arithmetic; only the last
  // step of a row can run past its end and has an offset of its own.
  auto issue_dy = [&](int oy, float (&bv)[kMaxTSteps][2]) {
    const bool row_ok = oy < oy_end;
    const unsigned lane_off =
        (static_cast<unsigned>((n * g.out_rows + oy) * g.out_cols + q) *
             kFeatures + 32 * kp + l16) * 4u;
    const unsigned v_main = row_ok ? lane_off : kOobOffset;
    const unsigned v_last =
        row_ok && 4 * (n_tsteps - 1) + q < g.out_cols ? lane_off : kOobOffset;
#pragma unroll
    for (int t = 0; t < kMaxTSteps; ++t) {
      if (t < n_tsteps) {
        const unsigned v = t == n_tsteps - 1 ? v_last : v_main;
#pragma unroll
        for (int j = 0; j < 2; ++j)
          bv[t][j] = __builtin_bit_cast(
              float, __builtin_amdgcn_raw_buffer_load_b32(
                         dy_rsrc, v, (4 * t * kFeatures + 16 * j) * 4, 0));
      }
    }
  };
  // The A operands of a step are fetched during the step before it (fenced:
  // left alone, the compiler reads one operand, waits for it and issues two
  // matrix instructions, and the LDS latency shows every time).
  auto multiply_row = [&](int oy, const float (&bv)[kMaxTSteps][2]) {
    const float* base = lds + kStride * (oy - oy0) * kRowFloats;
    float a[2][kRhoBlocks];
#pragma unroll
    for (int b = 0; b < kRhoBlocks; ++b) a[0][b] = base[a_off[b]];
#pragma unroll
    for (int t = 0; t < kMaxTSteps; ++t) {
      if (t < n_tsteps) {
        __builtin_amdgcn_sched_barrier(0);
        if (t + 1 < kMaxTSteps) {
#pragma unroll
          for (int b = 0; b < kRhoBlocks; ++b)
            a[(t + 1) & 1][b] = base[a_off[b] + 24 * (t + 1)];
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int b = 0; b < kRhoBlocks; ++b)
#pragma unroll
          for (int j = 0; j < 2; ++j)
            acc[b][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(
                a[t & 1][b], bv[t][j], acc[b][j], 0, 0, 0);
      }
    }
  };

  float bv0[kMaxTSteps][2], bv1[kMaxTSteps][2];
  issue_dy(oy0 + ph, bv0);
  __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
  __syncthreads();  // the band's rows are in LDS
#define SNN_STEM_FILBK_STEP(cur, nxt)                                  \
  {                                                                    \
    if (i >= n_iter) break;                                            \
    __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));                          \
    if (i + 1 < n_iter) issue_dy(oy0 + ph + 2 * (i + 1), nxt);         \
    multiply_row(oy0 + ph + 2 * i, cur);                               \
    ++i;                                                               \
  }
  int i = 0;
  for (;;) {
    SNN_STEM_FILBK_STEP(bv0, bv1)
    SNN_STEM_FILBK_STEP(bv1, bv0)
  }
#undef SNN_STEM_FILBK_STEP

  // the two row parities meet in LDS (the input rows are no longer needed)
  __syncthreads();
  constexpr int kWaveAcc = kRhoBlocks * 2 * 4 * 64;
  if (ph == 1) {
    float* dst = lds + (wave - 4) * kWaveAcc;
#pragma unroll
    for (int b = 0; b < kRhoBlocks; ++b)
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int v = 0; v < 4; ++v)
          dst[((b * 2 + j) * 4 + v) * 64 + lane] = acc[b][j][v];
  }
  __syncthreads();
  if (ph == 1) return;
  const float* src = lds + wave * kWaveAcc;
  float* out = part + static_cast<size_t>(blockIdx.x) * kPartFloats;
#pragma unroll
  for (int b = 0; b < kRhoBlocks; ++b)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        // accumulator element v of lane l: row 4 (l / 16) + v, column l % 16
        const int rho = 16 * (kRhoBlocks * rh + b) + 4 * q + v;
        const int k = 16 * (2 * kp + j) + l16;
        if (rho < kK)
          out[rho * kFeatures + k] =
              acc[b][j][v] + src[((b * 2 + j) * 4 + v) * 64 + lane];
      }
}

// dW = sum of the work-groups' partial filters: 4 consecutive float4 x 64
// groups of partials per work-group (588 work-groups for the 147 x 64 filter,
// four partials per lane at 256 of them), the groups meeting through LDS in a
// fixed order.
__global__ void __launch_bounds__(256)
    stem_filter_backprop_reduce_kernel(const float4v* __restrict__ part,
                                       float4v* __restrict__ dw, int n_parts) {
  __shared__ float4v sums[64][4];
  const int o4 = threadIdx.x & 3, group = threadIdx.x >> 2;
  const int o = blockIdx.x * 4 + o4;
  float4v sum = {0.f, 0.f, 0.f, 0.f};
  for (int sp = group; sp < n_parts; sp += 64)
    sum += part[static_cast<size_t>(sp) * (kPartFloats / 4) + o];
  sums[group][o4] = sum;
  __syncthreads();
  // eight lanes per element add eight groups each, then one adds the eight
  __shared__ float4v sums8[8][4];
  if (group < 8) {
    sum = sums[8 * group][o4];
#pragma unroll
    for (int i = 1; i < 8; ++i) sum += sums[8 * group + i][o4];
    sums8[group][o4] = sum;
  }
  __syncthreads();
  if (group != 0) return;
  sum = sums8[0][o4];
#pragma unroll
  for (int i = 1; i < 8; ++i) sum += sums8[i][o4];
  dw[o] = sum;
}

// ---------------------------------------------------------------------------
// Input gradient of the same layer:
//   dX[n][2 oy + r - pad][2 ox + s - pad][c] += sum over k of dY[n][oy][ox][k] * W[r][s][c][k].
// Per block of 16 output pixels, Z[rho][pixel] = W[rho][.] * dY[pixel][.] (ten
// row blocks of 16 x 16 reduction steps of 4) is computed on the matrix cores
// and added straight into the band's input rows in LDS (the layout is the
// forward kernel's), so the [pixels][147] intermediate never
// reaches memory.  The filter is the B operand and stays in registers (wave
// w: row blocks 5 (w & 1) ..., 80 registers); reduction index 16 q + t sits
// in lane group q at step t, which makes both operands runs of 16 consecutive
// floats per lane.  At the end the band's rows are written out: rows no other band touches with
// plain stores, the five rows shared with each neighbouring band with float
// atomics into the zero-filled output (two addends, so the result does not
// depend on their order).

__global__ void __launch_bounds__(64 * kWaves)
    __attribute__((amdgpu_waves_per_eu(2, 2)))
    conv_stem_input_backprop_kernel(const float* __restrict__ dy,
                                    const float* __restrict__ w,
                                    float* __restrict__ dx, StemGeom g) {
  extern __shared__ __align__(16) float lds[];
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int q = lane >> 4;
  const int l16 = lane & 15;
  const int rh = wave & 1;
  const int n = blockIdx.x / g.n_bands;
  const int band = blockIdx.x % g.n_bands;
  const int oy0 = band * g.band;
  const int n_rows = min(g.band, g.out_rows - oy0);
  const int y_first = kStride * oy0 - g.pad_rows;

  const __amdgpu_buffer_rsrc_t dy_rsrc = make_rsrc(
      dy, static_cast<size_t>(g.batch) * g.out_rows * g.out_cols * kFeatures * 4);
  const __amdgpu_buffer_rsrc_t dx_rsrc = make_rsrc(
      dx, static_cast<size_t>(g.batch) * g.in_rows * g.in_cols * kCh * 4);

  for (int i = threadIdx.x; i < g.lds_rows * kRowFloats; i += 64 * kWaves)
    lds[i] = 0.f;

  // filter rows 16 (5 rh + b) + l16, reduction indices 16 q + t
  float wreg[kRhoBlocks][16];
#pragma unroll
  for (int b = 0; b < kRhoBlocks; ++b) {
    const int rho = 16 * (kRhoBlocks * rh + b) + l16;
#pragma unroll
    for (int t4 = 0; t4 < 4; ++t4) {
      float4v v = {0.f, 0.f, 0.f, 0.f};
      if (rho < kK)
        v = *reinterpret_cast<const float4v*>(w + rho * kFeatures + 16 * q +
                                              4 * t4);
#pragma unroll
      for (int e = 0; e < 4; ++e) wreg[b][4 * t4 + e] = v[e];
    }
  }
  // Pixels are the rows of the product and rho its columns: accumulator
  // element v of row block b belongs to pixel 4 q + v and this lane's rho, and
  // lands at row rho / 21, float rho % 21 + 6 (4 q + v) relative to (first LDS
  // row of the output row, pixel block).  The 64 lanes of one LDS add then hit
  // 64 different floats (with rho down the rows, lanes two pixels and three
  // lane groups apart met in the same float and an add took ~100 cycles).
  int z_off[kRhoBlocks];
#pragma unroll
  for (int b = 0; b < kRhoBlocks; ++b) {
    const int rho = 16 * (kRhoBlocks * rh + b) + l16;
    z_off[b] = rho < kK ? (rho / kRowK) * kRowFloats + rho % kRowK + 24 * q : -1;
  }

  const int n_pb = (g.out_cols + 15) >> 4;
  // dY of a block for this lane: pixel 16 pb + l16, features 16 q ... + 15
  auto issue_dy = [&](int row, int pb, bool live, float4v (&bv)[4]) {
    const int ox = 16 * pb + l16;
    const bool ok = live && row < n_rows && ox < g.out_cols;
    const unsigned off =
        (static_cast<unsigned>((n * g.out_rows + oy0 + row) * g.out_cols + ox) *
             kFeatures + 16 * q) * 4u;
#pragma unroll
    for (int t4 = 0; t4 < 4; ++t4)
      bv[t4] = __builtin_bit_cast(
          float4v, __builtin_amdgcn_raw_buffer_load_b128(
                       dy_rsrc, ok ? off : kOobOffset, 16 * t4, 0));
  };
  // Z of one block, added into the band's rows.  Plain read-add-write: the 64
  // lanes of an instruction hit 64 different floats, and the schedule below
  // keeps the waves' blocks apart.  (LDS float atomics measured ~180 cycles
  // per instruction, four times the rest of the kernel.)
  auto multiply_add = [&](int row, int pb, const float4v (&bv)[4]) {
    float4v acc[kRhoBlocks];
#pragma unroll
    for (int b = 0; b < kRhoBlocks; ++b) acc[b] = float4v{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int t = 0; t < 16; ++t)
#pragma unroll
      for (int b = 0; b < kRhoBlocks; ++b)
        acc[b] = __builtin_amdgcn_mfma_f32_16x16x4f32(bv[t >> 2][t & 3], wreg[b][t],
                                                      acc[b], 0, 0, 0);
    // A float one lane updates for pixel 4 q + v is another lane's for pixel
    // 4 q + v + 1 (two taps to the left), so the four v must stay in program
    // order (the LDS serves a wave's accesses in order): a compiler barrier
    // between the batches keeps them there.  (Not `volatile`: every volatile
    // access waits for all vector-memory loads in flight as well, the next
    // block's dY among them -- a round trip to memory per block.)  The five
    // row blocks of one v never meet (their rho differ by less than the 24
    // floats between lane groups, or sit in different LDS rows) and go as one
    // batch of reads and one of writes.
    float* base = lds + kStride * row * kRowFloats + 96 * pb;
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      float old[kRhoBlocks];
      asm volatile("" ::: "memory");
#pragma unroll
      for (int b = 0; b < kRhoBlocks; ++b)
        old[b] = base[(z_off[b] >= 0 ? z_off[b] : 0) + 6 * v];
      asm volatile("" ::: "memory");
#pragma unroll
      for (int b = 0; b < kRhoBlocks; ++b)
        if (z_off[b] >= 0) base[z_off[b] + 6 * v] = old[b] + acc[b][v];
    }
    asm volatile("" ::: "memory");
  };

  // A block (output row, pixel block) touches LDS rows 2 row ... 2 row + 6 and
  // floats 96 pb ... 96 pb + 110: blocks four rows or two pixel blocks apart
  // are disjoint.  A step gives the eight waves eight such slots -- rows
  // i + 4 m (m = 0 ... 3) x pixel blocks {2 cs, 2 cs + 1} or {4 + 2 cs,
  // 5 + 2 cs} -- and a barrier ends it; every slot is visited twice, once by a
  // wave of each half of the rho range.
  const int wj = wave >> 1;
  const int n_steps = 16 * ((n_rows + 15) >> 4);
  auto decode = [&](int st, int& row, int& pb0) {
    const int sub = st & 1, cs = (st >> 1) & 1, i = (st >> 2) & 3, rg = st >> 4;
    const int slot = 2 * wj + (rh ^ sub);
    row = 16 * rg + i + 4 * (slot >> 1);
    pb0 = 4 * (slot & 1) + 2 * cs;
  };
  auto issue_item = [&](int st, float4v (&bv)[2][4]) {
    int row, pb0;
    decode(st, row, pb0);
#pragma unroll
    for (int d = 0; d < 2; ++d)
      issue_dy(row, pb0 + d, st < n_steps && pb0 + d < n_pb, bv[d]);
  };
  auto do_item = [&](int st, const float4v (&bv)[2][4]) {
    int row, pb0;
    decode(st, row, pb0);
#pragma unroll
    for (int d = 0; d < 2; ++d)
      if (row < n_rows && pb0 + d < n_pb) multiply_add(row, pb0 + d, bv[d]);
  };

  float4v bv0[2][4], bv1[2][4];
  issue_item(0, bv0);
  __syncthreads();  // the band's rows are zero
#define SNN_STEM_INBK_STEP(cur, nxt)                    \
  {                                                     \
    if (st >= n_steps) break;                           \
    issue_item(st + 1, nxt);                            \
    __builtin_amdgcn_s_waitcnt(vmcnt_imm(8));           \
    do_item(st, cur);                                   \
    __syncthreads();                                    \
    ++st;                                               \
  }
  int st = 0;
  for (;;) {
    SNN_STEM_INBK_STEP(bv0, bv1)
    SNN_STEM_INBK_STEP(bv1, bv0)
  }
#undef SNN_STEM_INBK_STEP
  __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
  __syncthreads();

  // ---- write the band's rows ------------------------------------------------
  const int row_floats_in = g.in_cols * kCh;
  const int first_col = kCh * g.pad_cols;
  for (int row = wave; row < g.lds_rows; row += kWaves) {
    const int yy = y_first + row;
    if (yy < 0 || yy >= g.in_rows) continue;
    const bool shared = (band > 0 && row < kWin - kStride) ||
                        (band + 1 < g.n_bands && row >= kStride * g.band);
    const unsigned row_off =
        static_cast<unsigned>(n * g.in_rows + yy) *
        static_cast<unsigned>(row_floats_in) * 4u;
    for (int f = lane; f < row_floats_in; f += 64) {
      const float v = lds[row * kRowFloats + first_col + f];
      const unsigned off = row_off + static_cast<unsigned>(f) * 4u;
      if (shared)
        __builtin_amdgcn_raw_ptr_buffer_atomic_fadd_f32(v, dx_rsrc, off, 0, 0);
      else
        __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, v),
                                              dx_rsrc, off, 0, 0);
    }
  }
}

// Zeroes the rows of dX that the band kernel does not store: the kWin - kStride
// rows that two neighbouring bands share (both add into them with atomics)
// and the rows below the last band's reach (no window touches them).  Block
// (image x band, r): band b < n_bands - 1 clears shared row r of its lower
// edge, the last band every fifth row from its reach + r on.
__global__ void __launch_bounds__(256)
    stem_zero_rows_kernel(float* __restrict__ dx, StemGeom g) {
  const int n = blockIdx.x / g.n_bands;
  const int band = blockIdx.x % g.n_bands;
  const int row_floats = g.in_cols * kCh;
  const int first = kStride * (band + 1) * g.band - g.pad_rows;
  if (band + 1 < g.n_bands) {
    const int y = first + static_cast<int>(blockIdx.y);
    if (y < 0 || y >= g.in_rows) return;
    float* row = dx + (static_cast<size_t>(n) * g.in_rows + y) * row_floats;
    for (int i = threadIdx.x; i < row_floats; i += 256) row[i] = 0.f;
  } else {
    for (int y = first + (kWin - kStride) + static_cast<int>(blockIdx.y);
         y < g.in_rows; y += kWin - kStride) {
      if (y < 0) continue;
      float* row = dx + (static_cast<size_t>(n) * g.in_rows + y) * row_floats;
      for (int i = threadIdx.x; i < row_floats; i += 256) row[i] = 0.f;
    }
  }
}

}  // namespace

bool conv2d_stem_supports(const snn_hip_conv2d_params& p) {
  StemGeom g;
  return make_geom(p, &g);
}

namespace {
template <typename TY>
int launch_stem_forward(const float* x, const float* w, TY* y,
                        const snn_hip_conv2d_params& p, hipStream_t stream) {
  StemGeom g;
  if (!make_geom(p, &g)) return SNN_HIP_INVALID_ALGORITHM;
  const size_t lds_bytes =
      (static_cast<size_t>(g.lds_rows + 1) * g.row_floats + 64) * sizeof(float);
  static const hipError_t attr = hipFuncSetAttribute(
      reinterpret_cast<const void*>(conv_stem_7x7s2_kernel<TY>),
      hipFuncAttributeMaxDynamicSharedMemorySize,
      static_cast<int>(kMaxLdsBytes));
  (void)attr;
  KernelTimer timer(stream);
  hipLaunchKernelGGL(conv_stem_7x7s2_kernel<TY>,
                     dim3(static_cast<unsigned>(p.batch * g.n_bands)),
                     dim3(64 * kWaves), lds_bytes, stream, x, w, y, g);
  return SNN_HIP_OK;
}
}  // namespace

// The output must be 16-byte aligned (the loads need nothing beyond 4).
int launch_conv2d_stem_f32(const float* x, const float* w, float* y,
                           const snn_hip_conv2d_params& p,
                           hipStream_t stream) {
  return launch_stem_forward<float>(x, w, y, p, stream);
}

// fp32 input and filter, the output rounded to binary16 on the store (8-byte
// aligned).
int launch_conv2d_stem_f32_to_f16(const float* x, const float* w, _Float16* y,
                                  const snn_hip_conv2d_params& p,
                                  hipStream_t stream) {
  return launch_stem_forward<_Float16>(x, w, y, p, stream);
}

bool conv2d_stem_filter_backprop_supports(const snn_hip_conv2d_params& p) {
  StemGeom g;
  return make_geom(p, &g) && p.out_cols <= 4 * kMaxTSteps;
}

// dw 16-byte aligned.  The partial filters (one of 147 x 64 floats per
// work-group) live in a stream-ordered temporary.
int launch_conv2d_stem_filter_backprop_f32(const float* x, const float* dy,
                                           float* dw,
                                           const snn_hip_conv2d_params& p,
                                           hipStream_t stream) {
  StemGeom g;
  if (!make_geom(p, &g) || p.out_cols > 4 * kMaxTSteps)
    return SNN_HIP_INVALID_ALGORITHM;
  const unsigned n_groups = static_cast<unsigned>(p.batch * g.n_bands);
  void* ptr = nullptr;
  if (temp_malloc_async(&ptr, static_cast<size_t>(n_groups) * kPartFloats *
                                  sizeof(float),
                        stream) != hipSuccess)
    return SNN_HIP_ALLOCATION_PROBLEM;
  float* part = static_cast<float*>(ptr);
  // the band's rows, and at the end the accumulators of four waves
  const size_t lds_bytes = std::max(
      (static_cast<size_t>(g.lds_rows + 1) * g.row_floats + 64) * sizeof(float),
      static_cast<size_t>(4 * kRhoBlocks * 2 * 4 * 64) * sizeof(float));
  static const hipError_t attr = hipFuncSetAttribute(
      reinterpret_cast<const void*>(conv_stem_filter_backprop_kernel),
      hipFuncAttributeMaxDynamicSharedMemorySize,
      static_cast<int>(kMaxLdsBytes));
  (void)attr;
  {
    KernelTimer timer(stream);
    hipLaunchKernelGGL(conv_stem_filter_backprop_kernel, dim3(n_groups),
                       dim3(64 * kWaves), lds_bytes, stream, x, dy, part, g);
  }
  static_assert(kPartFloats % 16 == 0, "whole groups of 4 float4");
  hipLaunchKernelGGL(stem_filter_backprop_reduce_kernel,
                     dim3(kPartFloats / 16), dim3(256), 0, stream,
                     reinterpret_cast<const float4v*>(part),
                     reinterpret_cast<float4v*>(dw), static_cast<int>(n_groups));
  const hipError_t err = hipGetLastError();
  temp_free_async(part, stream);
  if (err != hipSuccess) return report_hip_error(err, "stem filter backprop");
  return SNN_HIP_OK;
}

// (From 16 images of 112 output rows: below that the general path measured
// faster, 85 vs 92 us at batch 8.)
bool conv2d_stem_input_backprop_supports(const snn_hip_conv2d_params& p) {
  StemGeom g;
  return make_geom(p, &g) &&
         static_cast<long>(p.batch) * p.out_rows >= 8 * kMinOutputRows &&
         (static_cast<size_t>(p.batch) * p.in_rows * p.in_cols * kCh) % 4 == 0;
}

// Input rows that two neighbouring bands both touch receive their two parts
// through float atomics into the zero-filled dX: two addends commute, so the
// sum does not depend on their order.  With bands of two output rows (a pitch
// of four input rows against a seven-row window) a row can belong to three
// bands, and three addends do not.
bool conv2d_stem_input_backprop_reproducible(const snn_hip_conv2d_params& p) {
  StemGeom g;
  return make_geom(p, &g) && (g.n_bands < 3 || kStride * g.band >= kWin - kStride);
}

// dy, filter and dx 16-byte aligned.
int launch_conv2d_stem_input_backprop_f32(const float* dy, const float* w,
                                          float* dx,
                                          const snn_hip_conv2d_params& p,
                                          hipStream_t stream) {
  StemGeom g;
  if (!conv2d_stem_input_backprop_supports(p) || !make_geom(p, &g))
    return SNN_HIP_INVALID_ALGORITHM;
  hipLaunchKernelGGL(stem_zero_rows_kernel,
                     dim3(static_cast<unsigned>(p.batch * g.n_bands),
                          kWin - kStride),
                     dim3(256), 0, stream, dx, g);
  const size_t lds_bytes =
      (static_cast<size_t>(g.lds_rows + 1) * g.row_floats + 64) * sizeof(float);
  static const hipError_t attr = hipFuncSetAttribute(
      reinterpret_cast<const void*>(conv_stem_input_backprop_kernel),
      hipFuncAttributeMaxDynamicSharedMemorySize,
      static_cast<int>(kMaxLdsBytes));
  (void)attr;
  KernelTimer timer(stream);
  hipLaunchKernelGGL(conv_stem_input_backprop_kernel,
                     dim3(static_cast<unsigned>(p.batch * g.n_bands)),
                     dim3(64 * kWaves), lds_bytes, stream, dy, w, dx, g);
  return SNN_HIP_OK;
}

}  // namespace snn
