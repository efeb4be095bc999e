// Row-major fp32 GEMM  Y[m][n] = X[m][k] * W[k][n]  for short reductions
// (k = 64, 128, 256 or 512) with the filter held in registers: the 1x1 stride-1
// convolutions of the ResNet bottlenecks (src/conv2d/... Matmul algorithm,
// include/portdnn/conv2d/launch.h:59-118 with a 1x1 window) and row-major
// matmul of that shape (src/matmul/kernels.h:26-133).
//
// 256 persistent work-groups of 8 waves, one per CU.  A work-group owns a
// slice of 128 * FB features for its whole life: wave w keeps
// W[0..k)[n0 + 16 * FB * w ...) as MFMA operands in FB * k / 4 registers, read
// from memory once.  The work-groups of a feature slice walk the pixel tiles
// (16 * PB consecutive rows of X, i.e. one contiguous run of bytes) in
// round-robin order; a tile goes from memory into LDS with
// `buffer_load ... lds` (no registers, 1 KiB per instruction, one or two
// instructions per wave), three tiles in rotation, one barrier per tile.
// Per tile a wave issues PB * k / 16 ds_read_b128, PB * FB * k / 4
// v_mfma_f32_16x16x4_f32 and PB * FB 16-byte stores, and nothing else but
// address increments: with features as the matrix instruction's rows and
// pixels as its columns a lane ends with four consecutive features of one
// pixel.
//
// LDS layout of a tile: pixel-major, the 16-byte pieces of a pixel's k values
// XOR-swizzled with pixel % 8 so that the 16 lanes of a ds_read_b128 (16
// pixels, same k) fall on 8 different bank groups.  The swizzle is applied on
// the way in: an LDS-direct load writes lane i to base + 16 * i, but each lane
// chooses the global address it fetches.
//
// Reduction order inside an output: k = 16 * G + 4 * q + s for matrix
// instruction 4 * G + s and lane quarter q, summed by the matrix unit over q
// and accumulated over (G, s) in order.
#include "snn_kernels.h"

namespace snn {
namespace {

typedef float float4v __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) void* lds_ptr;

constexpr int kWaves = 8;
// The output is written once: stream it (slc) -- unless it is larger than the
// 256 MiB last-level cache, where ordinary stores measured 3-6 %
// faster (the launcher decides: stream_stores).
constexpr int kStoreAux = 2;
constexpr size_t kStreamStoreMaxBytes = size_t{256} << 20;
constexpr int kGroups = 2048 / kWaves;  // persistent work-groups: 8 waves per CU
constexpr unsigned kOobOffset = 0x7FFFFFF0u;  // beyond every buffer's range
constexpr size_t kMaxBufferBytes = 0x7FFFFFF0u;

__device__ inline __amdgpu_buffer_rsrc_t make_rsrc(const void* p,
                                                   size_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0,
                                           static_cast<unsigned>(bytes),
                                           0x00020000);
}

// vmcnt(n) alone (expcnt and lgkmcnt left at their maxima), n < 64: the
// counter's low four bits sit in bits 3:0, its high two in bits 15:14.
constexpr int vmcnt_imm(int n) {
  return 0x0F70 | (n & 15) | ((n >> 4) << 14);
}

// (The kernels proper are the plain functions below: the compiler drops the
// host side of a kernel *template* whose body names the LDS-direct load.)
//
// NS = 2: slices of 64 * FB features for filters with too few features for
// eight waves (n = 64): waves 0-3 and 4-7 hold the same four feature blocks
// and take the lower and the upper half of a tile of 32 * PB pixels.
// TRANSW: W is stored n x k (k contiguous) -- the 1x1 input gradient
// dX[m][c] = sum_k dY[m][k] * W[c][k] with the HWCF filter as it is; only the
// one-off filter load differs.
template <int KSTEPS, int PB, int FB, bool EPI, int NS, bool TRANSW>
__device__ __forceinline__ void gemm_wreg_body(
    const float* __restrict__ x, const float* __restrict__ w,
    float* __restrict__ y, int m, int n, int n_cols, int m_tiles,
    int cols_by_xcd, int stream_stores, const float* __restrict__ bias,
    int relu) {
  constexpr int K = 4 * KSTEPS;
  constexpr int TP = 16 * PB * NS;                // pixels per tile
  constexpr int FW = kWaves / NS;                 // waves along the features
  constexpr int TILE_FLOATS = TP * K;
  constexpr int TILE_BYTES = TILE_FLOATS * 4;
  constexpr int ROUNDS = TILE_BYTES / (1024 * kWaves);  // loads per wave and tile
  constexpr int STORES = PB * FB;                 // stores per wave and tile
  constexpr int PIECES_PER_PIXEL = K / 4;
  static_assert(TILE_BYTES % (1024 * kWaves) == 0, "whole load rounds");
  static_assert(2 * STORES + ROUNDS < 64, "vmcnt immediate");
  // three tiles in rotation; separate objects, so that the compiler's
  // bookkeeping ties a read to the loads of its own stage only
  __shared__ __align__(16) float s0[TILE_FLOATS];
  __shared__ __align__(16) float s1[TILE_FLOATS];
  __shared__ __align__(16) float s2[TILE_FLOATS];

  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int q = lane >> 4;    // lane quarter: reduction sub-index
  const int l16 = lane & 15;  // feature row (filter operand) / pixel column
  // Work-groups b, b + 8, ... share an XCD (and its L2).  Either the n_cols
  // groups that read one pixel tile are neighbours there (each XCD then
  // fetches an eighth of X and all of W), or -- cols_by_xcd, for filters larger
  // than X -- an XCD holds n_cols / 8 feature slices and every worker of each
  // (an eighth of W and all of X, which its L2 keeps).
  const int xcd = blockIdx.x & 7;
  const int j = blockIdx.x >> 3;
  const int workers = kGroups / n_cols;
  int col, tile;
  if (cols_by_xcd) {
    const int per_xcd = n_cols >> 3;
    col = xcd * per_xcd + j % per_xcd;
    tile = j / per_xcd;
  } else {
    col = j % n_cols;
    tile = (j / n_cols) * 8 + xcd;
  }
  const int wf = wave % FW, wp = wave / FW;
  const int n0 = (col * FW + wf) * 16 * FB;

  const __amdgpu_buffer_rsrc_t x_rsrc =
      make_rsrc(x, static_cast<size_t>(m) * K * 4);
  const __amdgpu_buffer_rsrc_t y_rsrc =
      make_rsrc(y, static_cast<size_t>(m) * n * 4);

  // The filter slice of this wave, in matrix-operand order: buffer loads
  // whose lane part is one register and whose step part is a scalar offset
  // (a pointer per load would be 2 K / 4 address registers: the compiler
  // spilled them and waited on the way).  W stored n x k gives the four steps
  // of a group with one 16-byte load.
  const __amdgpu_buffer_rsrc_t w_rsrc =
      make_rsrc(w, static_cast<size_t>(K) * n * 4);
  float wreg[FB][KSTEPS];
#pragma unroll
  for (int fb = 0; fb < FB; ++fb) {
    if (TRANSW) {
      const unsigned voff =
          static_cast<unsigned>((n0 + 16 * fb + l16) * K + 4 * q) * 4u;
#pragma unroll
      for (int g = 0; g < KSTEPS / 4; ++g) {
        const float4v v = __builtin_bit_cast(
            float4v, __builtin_amdgcn_raw_buffer_load_b128(w_rsrc, voff,
                                                           64 * g, 0));
#pragma unroll
        for (int s = 0; s < 4; ++s) wreg[fb][4 * g + s] = v[s];
      }
    } else {
      const unsigned voff =
          static_cast<unsigned>(4 * q * n + n0 + 16 * fb + l16) * 4u;
#pragma unroll
      for (int g = 0; g < KSTEPS / 4; ++g)
#pragma unroll
        for (int s = 0; s < 4; ++s)
          wreg[fb][4 * g + s] = __builtin_bit_cast(
              float, __builtin_amdgcn_raw_buffer_load_b32(
                         w_rsrc, voff,
                         static_cast<unsigned>((16 * g + s) * n) * 4u, 0));
    }
  }
  float4v bias4[FB];
  if (EPI) {
#pragma unroll
    for (int fb = 0; fb < FB; ++fb) {
      bias4[fb] = float4v{0.f, 0.f, 0.f, 0.f};
      if (bias != nullptr) {
        const float* b = bias + n0 + 16 * fb + 4 * q;
        bias4[fb] = float4v{b[0], b[1], b[2], b[3]};
      }
    }
  }

  // LDS piece p = round * 512 + wave * 64 + lane of a tile holds the k piece
  // (p % PIECES_PER_PIXEL) ^ (pixel % 8) of pixel p / PIECES_PER_PIXEL.
  unsigned src_off[ROUNDS];
#pragma unroll
  for (int r = 0; r < ROUNDS; ++r) {
    const int p = r * 64 * kWaves + wave * 64 + lane;
    const int pixel = p / PIECES_PER_PIXEL;
    const int piece = (p % PIECES_PER_PIXEL) ^ (pixel & 7);
    src_off[r] = static_cast<unsigned>(pixel * K + 4 * piece) * 4u;
  }
  auto issue = [&](float* stage, int t) {
    // a tile past the end is out of the buffer's range: zeros, no traffic
    const unsigned base = static_cast<unsigned>(t) * TILE_BYTES;
#pragma unroll
    for (int r = 0; r < ROUNDS; ++r)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(
          x_rsrc, (lds_ptr)(stage + (r * 64 * kWaves + wave * 64) * 4), 16,
          t < m_tiles ? base + src_off[r] : kOobOffset, 0, 0, 0);
  };
  // byte offsets of this lane's operand pieces in a stage, and of its outputs
  unsigned read_off[PB];
#pragma unroll
  for (int pb = 0; pb < PB; ++pb)
    read_off[pb] = static_cast<unsigned>((16 * (wp * PB + pb) + l16) * K) * 4u;
  const unsigned swz = static_cast<unsigned>(l16 & 7);
  const unsigned out_lane =
      static_cast<unsigned>((16 * wp * PB + l16) * n + n0 + 4 * q) * 4u;
  const unsigned out_tile_bytes = static_cast<unsigned>(TP * n) * 4u;

  auto compute = [&](const float* stage, int t) {
    float4v acc[PB][FB];
#pragma unroll
    for (int pb = 0; pb < PB; ++pb)
#pragma unroll
      for (int fb = 0; fb < FB; ++fb) acc[pb][fb] = float4v{0.f, 0.f, 0.f, 0.f};
    const char* sb = reinterpret_cast<const char*>(stage);
    // operand pieces are fetched one group of four matrix instructions ahead
    float4v xf[2][PB];
    auto fetch = [&](int g, float4v (&dst)[PB]) {
#pragma unroll
      for (int pb = 0; pb < PB; ++pb)
        dst[pb] = *reinterpret_cast<const float4v*>(
            sb + read_off[pb] + ((static_cast<unsigned>(4 * g + q) ^ swz) << 4));
    };
    fetch(0, xf[0]);
#pragma unroll
    for (int g = 0; g < KSTEPS / 4; ++g) {
      if (g + 1 < KSTEPS / 4) fetch(g + 1, xf[(g + 1) & 1]);
#pragma unroll
      for (int s = 0; s < 4; ++s)
#pragma unroll
        for (int pb = 0; pb < PB; ++pb)
#pragma unroll
          for (int fb = 0; fb < FB; ++fb)
            acc[pb][fb] = __builtin_amdgcn_mfma_f32_16x16x4f32(
                wreg[fb][4 * g + s], xf[g & 1][pb][s], acc[pb][fb], 0, 0, 0);
    }
    // rows past m fall outside the buffer's range and are dropped
    const unsigned base = static_cast<unsigned>(t) * out_tile_bytes + out_lane;
#pragma unroll
    for (int pb = 0; pb < PB; ++pb)
#pragma unroll
      for (int fb = 0; fb < FB; ++fb) {
        float4v v = acc[pb][fb];
        if (EPI) {
          v += bias4[fb];
          if (relu) {
            v.x = fmaxf(v.x, 0.f); v.y = fmaxf(v.y, 0.f);
            v.z = fmaxf(v.z, 0.f); v.w = fmaxf(v.w, 0.f);
          }
        }
        const unsigned off =
            base + static_cast<unsigned>(16 * pb * n + 16 * fb) * 4u;
        if (stream_stores)
          __builtin_amdgcn_raw_buffer_store_b128(v, y_rsrc, off, 0, kStoreAux);
        else
          __builtin_amdgcn_raw_buffer_store_b128(v, y_rsrc, off, 0, 0);
      }
  };

  // Vector-memory operations retire in order.  When step t waits for the
  // loads of tile t, the operations issued after them are the stores of tile
  // t - 2, the loads of tile t + 1 and the stores of tile t - 1: that many may
  // stay in flight.  Every step issues its loads and stores whether or not the
  // tile exists, so the count holds; the first two tiles are waited for in
  // full before the loop (with the filter), where it would not.
  constexpr int kInFlight = ROUNDS + 2 * STORES;
#define SNN_WREG_STEP(cur, nxt)                          \
  {                                                      \
    if (tile >= m_tiles) break;                          \
    __builtin_amdgcn_sched_barrier(0);                   \
    __builtin_amdgcn_s_waitcnt(vmcnt_imm(kInFlight));    \
    __builtin_amdgcn_s_barrier();                        \
    __builtin_amdgcn_sched_barrier(0);                   \
    issue(nxt, tile + 2 * workers);                      \
    compute(cur, tile);                                  \
    tile += workers;                                     \
  }
  issue(s0, tile);
  issue(s1, tile + workers);
  // The filter registers are pinned here so that their loads are in flight
  // together with the first two tiles (left alone, the compiler sinks the
  // loads below the wait, to their first use: two round trips to memory in a
  // row before the first matrix instruction).
#pragma unroll
  for (int fb = 0; fb < FB; ++fb)
#pragma unroll
    for (int i = 0; i < KSTEPS; ++i) asm volatile("" : "+v"(wreg[fb][i]));
  __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
  for (;;) {
    SNN_WREG_STEP(s0, s2)
    SNN_WREG_STEP(s1, s0)
    SNN_WREG_STEP(s2, s1)
  }
#undef SNN_WREG_STEP
  // loads of tiles past the end may still be on their way into LDS
  __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
}

struct Plan {
  int pb, fb, ns, n_cols, m_tiles;
};

// The tiling whose work-group tiles divide most evenly over the 256 groups.
bool make_plan(int m, int k, int n, Plan* plan, bool one_block = false) {
  if (k != 64 && k != 128 && k != 256 && k != 512) return false;
  double best = 0.0;
  bool found = false;
  for (int ns = 1; ns <= 2; ++ns) {
    for (int fb = one_block ? 1 : 2; fb >= 1; --fb) {
      const int slice = 16 * (kWaves / ns) * fb;
      if (n % slice != 0) continue;
      if (ns == 2 && fb != 1) continue;  // (built: one feature block per wave)
      const int n_cols = n / slice;
      if (n_cols > kGroups / 8 || (n_cols & (n_cols - 1)) != 0) continue;
      for (int pb = 2; pb >= 1; --pb) {
        if (ns == 2 && pb != 1) continue;
        const int tile_bytes = 16 * pb * ns * k * 4;
        if (tile_bytes % (1024 * kWaves) != 0) continue;
        if (3 * tile_bytes > 96 * 1024) continue;  // three tiles in LDS
        if (fb * (k / 4) > 128) continue;          // filter registers per lane
        const int m_tiles = ceil_div(m, 16 * pb * ns);
        const int workers = kGroups / n_cols;
        const int rounds = ceil_div(m_tiles, workers);
        if (rounds < 4) continue;  // too little work to amortise the filter load
        const double eff = static_cast<double>(m) /
                           (static_cast<double>(rounds) * workers * 16 * pb * ns);
        if (eff > best + 1e-9) {
          best = eff;
          *plan = Plan{pb, fb, ns, n_cols, m_tiles};
          found = true;
        }
      }
    }
    // eight feature waves whenever the feature count allows them
    if (found) break;
  }
  return found;
}

#define SNN_WREG_KERNEL_AS(KSTEPS, PB, FB, E, NS, TRANSW, NAME)                 \
  __global__ void __launch_bounds__(64 * kWaves)                               \
      __attribute__((amdgpu_waves_per_eu(2, 2)))                               \
      NAME(const float* __restrict__ x, const float* __restrict__ w,           \
           float* __restrict__ y, int m, int n, int n_cols, int m_tiles,       \
           int cols_by_xcd, int stream_stores, const float* __restrict__ bias, \
           int relu) {                                                         \
    gemm_wreg_body<KSTEPS, PB, FB, E != 0, NS, TRANSW>(                        \
        x, w, y, m, n, n_cols, m_tiles, cols_by_xcd, stream_stores, bias,      \
        relu);                                                                 \
  }
#define SNN_WREG_KERNEL(KSTEPS, PB, FB, E)      \
  SNN_WREG_KERNEL_AS(KSTEPS, PB, FB, E, 1, false, \
                     gemm_wreg_k##KSTEPS##_p##PB##_f##FB##_e##E)
#define SNN_WREG_KERNELS(KSTEPS, PB, FB) \
  SNN_WREG_KERNEL(KSTEPS, PB, FB, 0)     \
  SNN_WREG_KERNEL(KSTEPS, PB, FB, 1)
// (a 16-pixel tile of 64 reduction steps is half a load round; 32-pixel tiles
// of 512 steps do not fit LDS three times, nor two of its feature blocks the
// registers)
SNN_WREG_KERNELS(16, 2, 2) SNN_WREG_KERNELS(16, 2, 1)
SNN_WREG_KERNELS(32, 2, 2) SNN_WREG_KERNELS(32, 2, 1)
SNN_WREG_KERNELS(32, 1, 2) SNN_WREG_KERNELS(32, 1, 1)
SNN_WREG_KERNELS(64, 2, 2) SNN_WREG_KERNELS(64, 2, 1)
SNN_WREG_KERNELS(64, 1, 2) SNN_WREG_KERNELS(64, 1, 1)
SNN_WREG_KERNELS(128, 1, 1)
// 64-feature slices (four feature waves x two pixel halves)
SNN_WREG_KERNEL_AS(16, 1, 1, 0, 2, false, gemm_wreg_half_k16_e0)
SNN_WREG_KERNEL_AS(16, 1, 1, 1, 2, false, gemm_wreg_half_k16_e1)
SNN_WREG_KERNEL_AS(32, 1, 1, 0, 2, false, gemm_wreg_half_k32_e0)
SNN_WREG_KERNEL_AS(32, 1, 1, 1, 2, false, gemm_wreg_half_k32_e1)
SNN_WREG_KERNEL_AS(64, 1, 1, 0, 2, false, gemm_wreg_half_k64_e0)
SNN_WREG_KERNEL_AS(64, 1, 1, 1, 2, false, gemm_wreg_half_k64_e1)
// W stored n x k (the 1x1 input gradient): one feature block per wave
SNN_WREG_KERNEL_AS(16, 2, 1, 0, 1, true, gemm_wreg_t_k16_p2)
SNN_WREG_KERNEL_AS(32, 2, 1, 0, 1, true, gemm_wreg_t_k32_p2)
SNN_WREG_KERNEL_AS(32, 1, 1, 0, 1, true, gemm_wreg_t_k32_p1)
SNN_WREG_KERNEL_AS(64, 2, 1, 0, 1, true, gemm_wreg_t_k64_p2)
SNN_WREG_KERNEL_AS(64, 1, 1, 0, 1, true, gemm_wreg_t_k64_p1)
SNN_WREG_KERNEL_AS(16, 1, 1, 0, 2, true, gemm_wreg_t_half_k16)
SNN_WREG_KERNEL_AS(32, 1, 1, 0, 2, true, gemm_wreg_t_half_k32)
SNN_WREG_KERNEL_AS(64, 1, 1, 0, 2, true, gemm_wreg_t_half_k64)
#undef SNN_WREG_KERNELS
#undef SNN_WREG_KERNEL
#undef SNN_WREG_KERNEL_AS

using WregKernel = void (*)(const float*, const float*, float*, int, int, int,
                            int, int, int, const float*, int);

WregKernel pick_kernel(int k, const Plan& plan, bool epilogue,
                       bool transpose_w) {
  if (transpose_w) {
    // (k = 512 measured 3 % slower than the general kernel on the input
    // gradient of 28x28x128 -> 512 at batch 32; k <= 256 8 - 22 % faster)
    if (epilogue || plan.fb != 1 || k > 256) return nullptr;
    if (plan.ns == 2) {
      if (plan.pb != 1) return nullptr;
      return k == 64 ? gemm_wreg_t_half_k16
             : k == 128 ? gemm_wreg_t_half_k32
             : k == 256 ? gemm_wreg_t_half_k64
                        : nullptr;
    }
    if (k == 64 && plan.pb == 2) return gemm_wreg_t_k16_p2;
    if (k == 128) return plan.pb == 2 ? gemm_wreg_t_k32_p2 : gemm_wreg_t_k32_p1;
    if (k == 256) return plan.pb == 2 ? gemm_wreg_t_k64_p2 : gemm_wreg_t_k64_p1;
    return nullptr;
  }
  if (plan.ns == 2) {
    if (plan.pb != 1 || plan.fb != 1) return nullptr;
    if (k == 64) return epilogue ? gemm_wreg_half_k16_e1 : gemm_wreg_half_k16_e0;
    if (k == 128) return epilogue ? gemm_wreg_half_k32_e1 : gemm_wreg_half_k32_e0;
    if (k == 256) return epilogue ? gemm_wreg_half_k64_e1 : gemm_wreg_half_k64_e0;
    return nullptr;
  }
#define SNN_WREG_PICK(KSTEPS, PB, FB)                     \
  if (k == 4 * KSTEPS && plan.pb == PB && plan.fb == FB)  \
    return epilogue ? gemm_wreg_k##KSTEPS##_p##PB##_f##FB##_e1 \
                    : gemm_wreg_k##KSTEPS##_p##PB##_f##FB##_e0;
  SNN_WREG_PICK(16, 2, 2) SNN_WREG_PICK(16, 2, 1)
  SNN_WREG_PICK(32, 2, 2) SNN_WREG_PICK(32, 2, 1)
  SNN_WREG_PICK(32, 1, 2) SNN_WREG_PICK(32, 1, 1)
  SNN_WREG_PICK(64, 2, 2) SNN_WREG_PICK(64, 2, 1)
  SNN_WREG_PICK(64, 1, 2) SNN_WREG_PICK(64, 1, 1)
  SNN_WREG_PICK(128, 1, 1)
#undef SNN_WREG_PICK
  return nullptr;
}

}  // namespace

bool gemm_wreg_supports(int m, int k, int n, bool transpose_w) {
  Plan plan;
  return static_cast<size_t>(m) * max(k, n) * sizeof(float) <= kMaxBufferBytes &&
         make_plan(m, k, n, &plan, transpose_w) &&
         pick_kernel(k, plan, false, transpose_w) != nullptr;
}

// bias (one value per column, may be null) and relu are applied when
// `epilogue` is true.  Operands 16-byte aligned.
void launch_gemm_wreg(const float* x, const float* w, float* y, int m, int k,
                      int n, bool epilogue, const float* bias, bool relu,
                      hipStream_t stream, bool transpose_w) {
  Plan plan;
  if (!make_plan(m, k, n, &plan, transpose_w)) return;
  const WregKernel kernel = pick_kernel(k, plan, epilogue, transpose_w);
  if (kernel == nullptr) return;
  hipLaunchKernelGGL(kernel, dim3(kGroups), dim3(64 * kWaves), 0, stream, x, w,
                     y, m, n, plan.n_cols, plan.m_tiles,
                     plan.n_cols >= 8 && n > m ? 1 : 0,
                     static_cast<size_t>(m) * n * sizeof(float) <=
                             kStreamStoreMaxBytes
                         ? 1
                         : 0,
                     epilogue ? bias : nullptr, epilogue && relu ? 1 : 0);
}

}  // namespace snn
