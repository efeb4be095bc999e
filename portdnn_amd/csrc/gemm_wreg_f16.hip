// Row-major half-precision GEMM  Y[m][n] = X[m][k] * W[k][n]  (fp32
// accumulation) for short reductions, k = 64, 128, 256 or 512, with the filter
// held in registers: the 1x1 stride-1 convolutions of the ResNet bottlenecks
// (include/portdnn/conv2d/launch.h:59-118 with a 1x1 window) and row-major
// matmul of that shape (src/matmul/kernels.h:26-133) in binary16.
//
// Same scheme as the fp32 kernel of gemm_wreg.hip: 256 persistent work-groups
// of 8 waves, each owning a slice of 128 * FBW features for its whole life;
// pixel tiles (16 * PB consecutive rows of X, one contiguous run of bytes) go
// from memory into a ring of four LDS stages with `buffer_load ... lds`, one
// barrier per tile, and the waves do nothing per tile but ds_read_b128,
// v_mfma_f32_16x16x32_f16 and 16-byte stores.
//
// The filter operand.  The matrix instruction takes features as its rows: a
// lane supplies 8 consecutive reduction indices (k = 32 j + 8 q + 0..7 for
// instruction j and lane quarter q) of one feature.  W is feature-contiguous
// in memory, so a lane loads FBW consecutive features at each of its 8
// reduction indices (8 loads of 2 * FBW bytes per instruction j) and
// transposes the 8 x FBW block in registers into FBW operands.  Which feature
// is which matrix row is free: row i of feature block fb is feature
// n0 + FBW * i + fb, and since an output lane holds rows 4 q .. 4 q + 3 of every
// block it ends with the 4 * FBW consecutive features n0 + 4 * FBW * q ... of
// its pixel -- one or two 16-byte stores.
#include "snn_kernels.h"

namespace snn {
namespace {

typedef float float4v __attribute__((ext_vector_type(4)));
typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef unsigned int uint4v __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) void* lds_ptr;

constexpr int kWaves = 8;
constexpr int kGroups = 256;  // persistent work-groups: one per CU
constexpr int kStages = 4;    // LDS ring: three tiles in flight
// The output is written once: stream it (slc) -- unless it is larger than the
// 256 MiB last-level cache, where ordinary stores measured 3-6 %
// faster (the launcher decides: stream_stores).
constexpr int kStoreAux = 2;
constexpr size_t kStreamStoreMaxBytes = size_t{256} << 20;
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

template <int FBW>
struct FilterVec;
template <>
struct FilterVec<4> {
  using type = half4;
};
template <>
struct FilterVec<2> {
  using type = half2v;
};

// (The kernels proper are the plain functions below: the compiler drops the
// host side of a kernel *template* whose body names the LDS-direct load.)
// KS: matrix instructions per output block (k / 32); PB: 16-pixel blocks per
// tile; FBW: feature blocks per wave.
template <int KS, int PB, int FBW>
__device__ __forceinline__ void gemm_wreg_f16_body(
    const _Float16* __restrict__ x, const _Float16* __restrict__ w,
    _Float16* __restrict__ y, int m, int n, int n_cols, int m_tiles,
    int cols_by_xcd, int stream_stores) {
  constexpr int K = 32 * KS;
  constexpr int TP = 16 * PB;  // pixels per tile
  constexpr int TILE_HALVES = TP * K;
  constexpr int TILE_BYTES = TILE_HALVES * 2;
  constexpr int ROUNDS = TILE_BYTES / (1024 * kWaves);  // loads per wave and tile
  constexpr int STORE_VECS = FBW / 2;                   // 16-byte stores per block row
  constexpr int STORES = PB * STORE_VECS;               // stores per wave and tile
  constexpr int PIECES_PER_PIXEL = K / 8;
  static_assert(TILE_BYTES % (1024 * kWaves) == 0, "whole load rounds");
  constexpr int kInFlight = (kStages - 2) * ROUNDS + (kStages - 1) * STORES;
  static_assert(kInFlight < 64, "vmcnt immediate");
  // separate objects, so that the compiler's bookkeeping ties a read to the
  // loads of its own stage only
  __shared__ __align__(16) _Float16 s0[TILE_HALVES];
  __shared__ __align__(16) _Float16 s1[TILE_HALVES];
  __shared__ __align__(16) _Float16 s2[TILE_HALVES];
  __shared__ __align__(16) _Float16 s3[TILE_HALVES];

  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int q = lane >> 4;
  const int l16 = lane & 15;
  // Work-groups b, b + 8, ... share an XCD (and its L2): either the n_cols
  // groups that read one pixel tile are neighbours there, or (cols_by_xcd, for
  // filters larger than X) an XCD holds n_cols / 8 whole feature slices.
  const int xcd = blockIdx.x & 7;
  const int j8 = blockIdx.x >> 3;
  const int workers = kGroups / n_cols;
  int col, tile;
  if (cols_by_xcd) {
    const int per_xcd = n_cols >> 3;
    col = xcd * per_xcd + j8 % per_xcd;
    tile = j8 / per_xcd;
  } else {
    col = j8 % n_cols;
    tile = (j8 / n_cols) * 8 + xcd;
  }
  const int n0 = (col * kWaves + wave) * 16 * FBW;

  const __amdgpu_buffer_rsrc_t x_rsrc =
      make_rsrc(x, static_cast<size_t>(m) * K * 2);
  const __amdgpu_buffer_rsrc_t y_rsrc =
      make_rsrc(y, static_cast<size_t>(m) * n * 2);

  // the filter slice of this wave, transposed into matrix-operand order
  half8 wop[FBW][KS];
  {
    using Vec = typename FilterVec<FBW>::type;
    const _Float16* wp = w + n0 + FBW * l16;
#pragma unroll
    for (int j = 0; j < KS; ++j) {
      Vec v[8];
#pragma unroll
      for (int e = 0; e < 8; ++e)
        v[e] = *reinterpret_cast<const Vec*>(
            wp + static_cast<size_t>(32 * j + 8 * q + e) * n);
#pragma unroll
      for (int fb = 0; fb < FBW; ++fb)
#pragma unroll
        for (int e = 0; e < 8; ++e) wop[fb][j][e] = v[e][fb];
    }
  }

  // LDS piece p = round * 512 + wave * 64 + lane of a tile holds the 16-byte
  // k piece (p % PIECES_PER_PIXEL) ^ (pixel % 8) of pixel p / PIECES_PER_PIXEL.
  unsigned src_off[ROUNDS];
#pragma unroll
  for (int r = 0; r < ROUNDS; ++r) {
    const int p = r * 64 * kWaves + wave * 64 + lane;
    const int pixel = p / PIECES_PER_PIXEL;
    const int piece = (p % PIECES_PER_PIXEL) ^ (pixel & 7);
    src_off[r] = static_cast<unsigned>(pixel * K + 8 * piece) * 2u;
  }
  auto issue = [&](_Float16* stage, int t) {
    // a tile past the end is out of the buffer's range: zeros, no traffic
    const unsigned base = static_cast<unsigned>(t) * TILE_BYTES;
#pragma unroll
    for (int r = 0; r < ROUNDS; ++r)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(
          x_rsrc, (lds_ptr)(stage + (r * 64 * kWaves + wave * 64) * 8), 16,
          t < m_tiles ? base + src_off[r] : kOobOffset, 0, 0, 0);
  };
  unsigned read_off[PB];
#pragma unroll
  for (int pb = 0; pb < PB; ++pb)
    read_off[pb] = static_cast<unsigned>((16 * pb + l16) * K) * 2u;
  const unsigned swz = static_cast<unsigned>(l16 & 7);
  const unsigned out_lane =
      static_cast<unsigned>(l16 * n + n0 + 4 * FBW * q) * 2u;
  const unsigned out_tile_bytes = static_cast<unsigned>(TP * n) * 2u;

  auto compute = [&](const _Float16* stage, int t) {
    float4v acc[PB][FBW];
#pragma unroll
    for (int pb = 0; pb < PB; ++pb)
#pragma unroll
      for (int fb = 0; fb < FBW; ++fb) acc[pb][fb] = float4v{0.f, 0.f, 0.f, 0.f};
    const char* sb = reinterpret_cast<const char*>(stage);
    // operand pieces are fetched one matrix-instruction group ahead
    half8 xf[2][PB];
    auto fetch = [&](int j, half8 (&dst)[PB]) {
#pragma unroll
      for (int pb = 0; pb < PB; ++pb)
        dst[pb] = *reinterpret_cast<const half8*>(
            sb + read_off[pb] + ((static_cast<unsigned>(4 * j + q) ^ swz) << 4));
    };
    fetch(0, xf[0]);
#pragma unroll
    for (int j = 0; j < KS; ++j) {
      if (j + 1 < KS) fetch(j + 1, xf[(j + 1) & 1]);
#pragma unroll
      for (int pb = 0; pb < PB; ++pb)
#pragma unroll
        for (int fb = 0; fb < FBW; ++fb)
          acc[pb][fb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(
              wop[fb][j], xf[j & 1][pb], acc[pb][fb], 0, 0, 0);
    }
    // rows past m fall outside the buffer's range and are dropped
    const unsigned base = static_cast<unsigned>(t) * out_tile_bytes + out_lane;
#pragma unroll
    for (int pb = 0; pb < PB; ++pb) {
      // feature n0 + 4 * FBW * q + FBW * v + fb is component v of block fb
#pragma unroll
      for (int sv = 0; sv < STORE_VECS; ++sv) {
        half8 o;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const int f = 8 * sv + e;  // feature within the lane's run
          o[e] = static_cast<_Float16>(acc[pb][f % FBW][f / FBW]);
        }
        const unsigned off =
            base + static_cast<unsigned>(16 * pb * n + 8 * sv) * 2u;
        if (stream_stores)
          __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(uint4v, o),
                                                 y_rsrc, off, 0, kStoreAux);
        else
          __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(uint4v, o),
                                                 y_rsrc, off, 0, 0);
      }
    }
  };

  // Vector-memory operations retire in order.  When step t waits for the
  // loads of tile t, issued three steps earlier, the operations issued after
  // them are the stores of tiles t - 3 .. t - 1 and the loads of tiles t + 1
  // and t + 2: that many may stay in flight.  Every step issues its loads and
  // stores whether or not the tile exists, so the count holds; the first tiles
  // are waited for in full before the loop (with the filter), where it would
  // not.
#define SNN_WREG_STEP(cur, nxt)                          \
  {                                                      \
    if (tile >= m_tiles) break;                          \
    __builtin_amdgcn_sched_barrier(0);                   \
    __builtin_amdgcn_s_waitcnt(vmcnt_imm(kInFlight));    \
    __builtin_amdgcn_s_barrier();                        \
    __builtin_amdgcn_sched_barrier(0);                   \
    issue(nxt, tile + (kStages - 1) * workers);          \
    compute(cur, tile);                                  \
    tile += workers;                                     \
  }
  __builtin_amdgcn_sched_barrier(0);  // (the filter loads above go first)
  issue(s0, tile);
  issue(s1, tile + workers);
  issue(s2, tile + 2 * workers);
  __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
  for (;;) {
    SNN_WREG_STEP(s0, s3)
    SNN_WREG_STEP(s1, s0)
    SNN_WREG_STEP(s2, s1)
    SNN_WREG_STEP(s3, s2)
  }
#undef SNN_WREG_STEP
  // loads of tiles past the end may still be on their way into LDS
  __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
}

struct Plan {
  int pb, fbw, n_cols, m_tiles;
};

// The tiling whose work-group tiles divide most evenly over the 256 groups.
bool make_plan(int m, int k, int n, Plan* plan) {
  if (k != 64 && k != 128 && k != 256 && k != 512) return false;
  double best = 0.0;
  bool found = false;
  for (int fbw = 4; fbw >= 2; fbw -= 2) {
    const int slice = 16 * kWaves * fbw;
    if (n % slice != 0) continue;
    if (fbw * (k / 32) * 4 > 128) continue;  // filter registers per lane
    const int n_cols = n / slice;
    if (n_cols > kGroups / 8 || (n_cols & (n_cols - 1)) != 0) continue;
    for (int pb = 4; pb >= 1; pb >>= 1) {
      const int tile_bytes = 16 * pb * k * 2;
      if (pb == 4 && k != 64) continue;  // built for the shortest reduction only
      if (tile_bytes % (1024 * kWaves) != 0) continue;
      const int m_tiles = ceil_div(m, 16 * pb);
      const int workers = kGroups / n_cols;
      const int rounds = ceil_div(m_tiles, workers);
      if (rounds < 4) continue;  // too little work to amortise the filter load
      const double eff = static_cast<double>(m) /
                         (static_cast<double>(rounds) * workers * 16 * pb);
      if (eff > best + 1e-9) {
        best = eff;
        *plan = Plan{pb, fbw, n_cols, m_tiles};
        found = true;
      }
    }
  }
  return found;
}

#define SNN_WREG_F16_KERNEL(KS, PB, FBW)                                      \
  __global__ void __launch_bounds__(64 * kWaves)                              \
      __attribute__((amdgpu_waves_per_eu(2, 2)))                              \
      gemm_wreg_f16_k##KS##_p##PB##_f##FBW(                                   \
          const _Float16* __restrict__ x, const _Float16* __restrict__ w,     \
          _Float16* __restrict__ y, int m, int n, int n_cols, int m_tiles,    \
          int cols_by_xcd, int stream_stores) {                               \
    gemm_wreg_f16_body<KS, PB, FBW>(x, w, y, m, n, n_cols, m_tiles,           \
                                    cols_by_xcd, stream_stores);              \
  }
// (a load round is 8 KiB: 64 pixels of 64 reduction steps, 32 of 128; four
// feature blocks of 512 steps do not fit the registers)
SNN_WREG_F16_KERNEL(2, 4, 4) SNN_WREG_F16_KERNEL(2, 4, 2)
SNN_WREG_F16_KERNEL(4, 2, 4) SNN_WREG_F16_KERNEL(4, 2, 2)
SNN_WREG_F16_KERNEL(8, 2, 4) SNN_WREG_F16_KERNEL(8, 2, 2)
SNN_WREG_F16_KERNEL(8, 1, 4) SNN_WREG_F16_KERNEL(8, 1, 2)
SNN_WREG_F16_KERNEL(16, 2, 2) SNN_WREG_F16_KERNEL(16, 1, 2)
#undef SNN_WREG_F16_KERNEL

using WregKernel = void (*)(const _Float16*, const _Float16*, _Float16*, int,
                            int, int, int, int, int);

WregKernel pick_kernel(int k, const Plan& plan) {
#define SNN_WREG_PICK(KS, PB, FBW)                          \
  if (k == 32 * KS && plan.pb == PB && plan.fbw == FBW)     \
    return gemm_wreg_f16_k##KS##_p##PB##_f##FBW;
  SNN_WREG_PICK(2, 4, 4) SNN_WREG_PICK(2, 4, 2)
  SNN_WREG_PICK(4, 2, 4) SNN_WREG_PICK(4, 2, 2)
  SNN_WREG_PICK(8, 2, 4) SNN_WREG_PICK(8, 2, 2)
  SNN_WREG_PICK(8, 1, 4) SNN_WREG_PICK(8, 1, 2)
  SNN_WREG_PICK(16, 2, 2) SNN_WREG_PICK(16, 1, 2)
#undef SNN_WREG_PICK
  return nullptr;
}

}  // namespace

bool gemm_wreg_f16_supports(int m, int k, int n) {
  Plan plan;
  return static_cast<size_t>(m) * max(k, n) * sizeof(_Float16) <=
             kMaxBufferBytes &&
         make_plan(m, k, n, &plan) && pick_kernel(k, plan) != nullptr;
}

// Operands 16-byte aligned.
void launch_gemm_wreg_f16(const _Float16* x, const _Float16* w, _Float16* y,
                          int m, int k, int n, hipStream_t stream) {
  Plan plan;
  if (!make_plan(m, k, n, &plan)) return;
  const WregKernel kernel = pick_kernel(k, plan);
  if (kernel == nullptr) return;
  hipLaunchKernelGGL(kernel, dim3(kGroups), dim3(64 * kWaves), 0, stream, x, w,
                     y, m, n, plan.n_cols, plan.m_tiles,
                     plan.n_cols >= 8 && n > m ? 1 : 0,
                     static_cast<size_t>(m) * n * sizeof(_Float16) <=
                             kStreamStoreMaxBytes
                         ? 1
                         : 0);
}

}  // namespace snn
