// fp32 stride-1 convolution on MFMA (gfx950) for deep, small layers: the
// input rows of a tile in LDS as in conv2d_rowtile.hip, with the REDUCTION
// split over the eight waves of a work-group (forward, and the stride-1 input
// gradient as a forward convolution over dY with mirrored taps; the kernel
// behind the Tiled and Im2col tags where that one does not fit; portDNN:
// src/conv2d/tiled/kernels.h:99-190, src/conv2d/im2col/).
//
// A layer like 7x7x512 -> 512 at batch 32 has 1568 output pixels and 4608
// reduction steps: 98 x 32 blocks of 16 x 16 outputs for 1024 SIMDs.  Splitting
// the pixels or features of a work-group's tile over its waves, as the other
// kernel does, leaves a wave two to four blocks -- too few matrix instructions
// per filter load, per LDS tile and per barrier -- and splitting the reduction
// over work-groups means float atomics and several times the traffic.  Here
// every wave of a work-group owns ALL of the tile's blocks (FA feature blocks
// x PB pixel blocks, up to 28) and one eighth of the channels:
//
//   * wave w takes the 16-channel blocks w, w + 8, ...; for each it loads the
//     tile's input rows (halo and zero padding included) into its own LDS
//     buffer with LDS-direct buffer loads, waits for them alone -- no barrier:
//     nobody else reads that buffer -- and runs the filter taps over it,
//     4 FA PB matrix instructions (v_mfma_f32_16x16x4_f32) per tap for FA
//     filter loads straight from the HWCF tensor and PB ds_read_b128;
//   * the operands of the next tap are fetched while the current one is
//     multiplied; a wave that waits for its next tile leaves the matrix pipe
//     to the other wave of its SIMD;
//   * at the end the eight partial results meet in LDS, one feature block at
//     a time, and are added in wave order (reproducible, no atomics), with
//     bias and ReLU on the way out.
//
// Channels in multiples of 128, features of 16 FA.
#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <numeric>

#include "gemm_tile.h"
#include "snn_kernels.h"

namespace snn {
namespace {

using gemm::xcd_remap;

typedef float float4v __attribute__((ext_vector_type(4)));
typedef unsigned int uint4v __attribute__((ext_vector_type(4)));
constexpr unsigned kOob = 0x7FFFFFF0u;
constexpr size_t kMaxBufferBytes = 0x7FFFFFF0u;
constexpr size_t kMaxLdsBytes = 160 * 1024;
constexpr int kKC = 16;                   // channels per LDS tile
constexpr int kSlotBytes = kKC * 4 + 16;  // one pad piece: 5 pieces per slot
constexpr int kWaves = 8;                 // shares of the reduction
constexpr int kComputeUnits = 256;
constexpr int kMaxBlocks = 16;           // 1 KB blocks of a wave's tile

struct SplitTile {
  int batch, in_rows, in_cols, channels, features;
  int out_rows, out_cols;
  int win_rows, win_cols, pad_rows, pad_cols;
  int tile_pixels;   // output pixels (flattened n, y, x) per work-group
  int total_pixels;  // batch * out_rows * out_cols
  int padded_rows;   // Hp = out_rows + win_rows - 1: padded rows per image
  int halo_cols;     // Wh = out_cols + win_cols - 1
  int n_slots;       // LDS pixel slots per tile = lds rows * Wh
  int n_fslices;     // features / (16 * FA)
};

__device__ inline __amdgpu_buffer_rsrc_t make_rsrc(const void* p,
                                                   unsigned bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, bytes,
                                           0x00020000);
}

// FA: feature blocks of 16, PB: pixel blocks of 16 -- every wave holds all of
// them.  TRANSPOSED: the filter operand is w[taps - 1 - tap][f][c] of an HWCF
// tensor whose channel count is this launch's feature count (input gradient).
template <int FA, int PB, bool TRANSPOSED>
__global__ void __launch_bounds__(64 * kWaves)
    conv_rowsplit_f32_kernel(const float* __restrict__ src,
                             const float* __restrict__ wgt,
                             float* __restrict__ dst, SplitTile g,
                             unsigned src_bytes, unsigned wgt_bytes,
                             unsigned dst_bytes, unsigned n_groups,
                             const float* __restrict__ bias, int relu) {
  constexpr int NT = 64 * kWaves;
  extern __shared__ __align__(16) unsigned char lds[];
  typedef __attribute__((address_space(3))) void* lds_ptr;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const unsigned group = xcd_remap(blockIdx.x, n_groups);
  const int tile = static_cast<int>(group / g.n_fslices);
  const int fslice = static_cast<int>(group % g.n_fslices);

  const int pixel0 = tile * g.tile_pixels;  // first flattened output pixel
  const int n_pixels = min(g.tile_pixels, g.total_pixels - pixel0);
  // Padded-row coordinate of the first LDS row: image * Hp + padded row.
  const int row0 = pixel0 / g.out_cols;  // flattened (image, row)
  const int first_padded =
      (row0 / g.out_rows) * g.padded_rows + row0 % g.out_rows;

  // 1 KB blocks per tile, and the slots they reach into
  const int n_blocks = (g.n_slots * kSlotBytes + 1023) / 1024;
  const int n_table = n_blocks * 1024 / kSlotBytes + 1;
  const int buf_bytes = n_blocks * 1024;
  // the buffers of the eight waves; behind them the offset table.  The
  // partial results are added up in the same memory at the end.
  const int work_bytes = max(kWaves * buf_bytes, kWaves * PB * 1024);
  unsigned char* const my_buf = lds + wave * buf_bytes;
  unsigned* const table = reinterpret_cast<unsigned*>(lds + work_bytes);

  // Global byte offset of channel 0 of every pixel slot (kOob for padding
  // and for the slots that only fill up the last block).
  for (int slot = tid; slot < n_table; slot += NT) {
    const int lrow = slot / g.halo_cols;
    const int hx = slot - lrow * g.halo_cols;
    const int padded = first_padded + lrow;
    const int n = padded / g.padded_rows;
    const int iy = padded - n * g.padded_rows - g.pad_rows;
    const int ix = hx - g.pad_cols;
    const bool ok = slot < g.n_slots && n < g.batch &&
                    static_cast<unsigned>(iy) <
                        static_cast<unsigned>(g.in_rows) &&
                    static_cast<unsigned>(ix) < static_cast<unsigned>(g.in_cols);
    table[slot] =
        ok ? static_cast<unsigned>(((n * g.in_rows + iy) * g.in_cols + ix) *
                                   g.channels) * 4u
           : kOob;
  }
  __syncthreads();

  const __amdgpu_buffer_rsrc_t src_rsrc = make_rsrc(src, src_bytes);
  const __amdgpu_buffer_rsrc_t wgt_rsrc = make_rsrc(wgt, wgt_bytes);

  // The loads of one channel block into this wave's buffer: lane l fills
  // bytes 16 l .. 16 l + 15 of each 1 KB block, which belong to piece
  // (position % slot bytes) / 16 of slot position / slot bytes; the pad piece
  // of a slot and padding pixels load from out of range (zeros).  What a lane
  // fetches for a block does not depend on the channel block -- that offset
  // travels in the scalar offset (not range-checked; the vector offset is) --
  // so the vector offsets are worked out once and a tile is kMaxBlocks
  // back-to-back load instructions.
  unsigned tile_voff[kMaxBlocks];
#pragma unroll
  for (int block = 0; block < kMaxBlocks; ++block) {
    tile_voff[block] = kOob;
    if (block < n_blocks) {
      const int pos = block * 1024 + lane * 16;
      const int slot = pos / kSlotBytes;
      const int piece = (pos - slot * kSlotBytes) >> 4;
      const unsigned base = table[slot];
      if (piece < kKC / 4 && base != kOob)
        tile_voff[block] = base + static_cast<unsigned>(piece) * 16u;
    }
  }
  auto start_tile = [&](int chunk) {
    const unsigned coff = static_cast<unsigned>(chunk) * (kKC * 4u);
#pragma unroll
    for (int block = 0; block < kMaxBlocks; ++block)
      if (block < n_blocks)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(
            src_rsrc, (lds_ptr)(my_buf + block * 1024), 16, tile_voff[block],
            coff, 0, 0);
  };

  // LDS byte offset (tap (0,0), channel 4 q of the block) of this lane's
  // pixel in each pixel block (lanes past the tile multiply slot 0).
  const int l16 = lane & 15;
  const int q = lane >> 4;
  int lane_base[PB];
#pragma unroll
  for (int j = 0; j < PB; ++j) {
    const int pq = j * 16 + l16;
    lane_base[j] = q * 16;
    if (pq < n_pixels) {
      const int m = pixel0 + pq;
      const int orow = m / g.out_cols;
      const int x = m - orow * g.out_cols;
      const int n = orow / g.out_rows;
      const int lrow = n * g.padded_rows + (orow - n * g.out_rows) -
                       first_padded;
      lane_base[j] = (lrow * g.halo_cols + x) * kSlotBytes + q * 16;
    }
  }

  const int taps = g.win_rows * g.win_cols;
  const int n_chunks = g.channels / kKC;
  const int f0 = fslice * 16 * FA;
  // Filter operand of feature block i at a step.  Forward: w[tap][c0 + 4 q +
  // t][f0 + 16 i + l16], four loads a row of the filter apart.  Input
  // gradient: w[taps - 1 - tap][f0 + 16 i + l16][c0 + 4 q .. + 3], one load.
  // The lane's part of the address is fixed, the step's part is wave-uniform
  // and travels in the scalar offset.
  const unsigned a_lane =
      TRANSPOSED
          ? static_cast<unsigned>((f0 + l16) * g.channels + 4 * q) * 4u
          : static_cast<unsigned>(4 * q * g.features + f0 + l16) * 4u;
  const unsigned a_row = static_cast<unsigned>(g.features) * 4u;
  const unsigned a_block =
      TRANSPOSED ? static_cast<unsigned>(16 * g.channels) * 4u : 64u;
  auto load_a = [&](float4v (&frag)[FA], int tap, int chunk) {
    if (TRANSPOSED) {
      const unsigned soff =
          static_cast<unsigned>((taps - 1 - tap) * g.features * g.channels +
                                chunk * kKC) * 4u;
#pragma unroll
      for (int i = 0; i < FA; ++i)
        frag[i] = __builtin_bit_cast(
            float4v, __builtin_amdgcn_raw_buffer_load_b128(
                         wgt_rsrc, a_lane + static_cast<unsigned>(i) * a_block,
                         soff, 0));
    } else {
      const unsigned soff =
          static_cast<unsigned>(tap * g.channels + chunk * kKC) * a_row;
#pragma unroll
      for (int i = 0; i < FA; ++i)
#pragma unroll
        for (int t = 0; t < 4; ++t)
          frag[i][t] = __builtin_bit_cast(
              float, __builtin_amdgcn_raw_buffer_load_b32(
                         wgt_rsrc, a_lane + static_cast<unsigned>(i) * a_block,
                         soff + static_cast<unsigned>(t) * a_row, 0));
    }
  };
  auto read_b = [&](float4v (&b)[PB], int offset) {
#pragma unroll
    for (int j = 0; j < PB; ++j)
      b[j] = *reinterpret_cast<const float4v*>(my_buf + lane_base[j] + offset);
  };

  float4v acc[FA][PB];
#pragma unroll
  for (int i = 0; i < FA; ++i)
#pragma unroll
    for (int j = 0; j < PB; ++j) acc[i][j] = float4v{0.f, 0.f, 0.f, 0.f};

  // Filter fragments run one step ahead of the matrix instructions, across
  // this wave's channel blocks (their addresses do not depend on LDS).  The
  // step past the wave's last one loads the start of the filter (never used).
  float4v a_cur[FA];
  int a_tap = 0, a_chunk = wave;
  auto fetch_a = [&](float4v (&frag)[FA]) {
    const bool ok = a_chunk < n_chunks;
    load_a(frag, ok ? a_tap : 0, ok ? a_chunk : 0);
    if (++a_tap == taps) {
      a_tap = 0;
      a_chunk += kWaves;
    }
  };
  fetch_a(a_cur);
  start_tile(wave);
  for (int chunk = wave; chunk < n_chunks; chunk += kWaves) {
    float4v b_cur[PB], b_nxt[PB];
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): the tile is in LDS
    __builtin_amdgcn_sched_barrier(0);
    read_b(b_cur, 0);
    int r = 0, c = 0;
    for (int tap = 0; tap < taps; ++tap) {
      const bool more = tap + 1 < taps;
      if (++c == g.win_cols) {
        c = 0;
        ++r;
      }
      float4v a_new[FA];
      fetch_a(a_new);
      if (more) {
        read_b(b_nxt, (r * g.halo_cols + c) * kSlotBytes);
      } else if (chunk + kWaves < n_chunks) {
        // The last tap's pixel operands are in registers (they were read a
        // step ago): the buffer is free, and the next channel block's tile
        // loads while the last tap is multiplied.
        __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
        __builtin_amdgcn_sched_barrier(0);
        start_tile(chunk + kWaves);
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int i = 0; i < FA; ++i)
#pragma unroll
          for (int j = 0; j < PB; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(
                a_cur[i][t], b_cur[j][t], acc[i][j], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < FA; ++i) a_cur[i] = a_new[i];
      if (more) {
#pragma unroll
        for (int j = 0; j < PB; ++j) b_cur[j] = b_nxt[j];
      }
    }
  }

  // ---- the eight shares meet in LDS, one feature block at a time -----------
  // Thread e < 64 PB adds up, in wave order, the four values lane e % 64 holds
  // of pixel block e / 64 (features 4 q .. 4 q + 3 of pixel l16), and stores
  // them.
  const __amdgpu_buffer_rsrc_t dst_rsrc = make_rsrc(dst, dst_bytes);
  float4v* const part = reinterpret_cast<float4v*>(lds);
  const int e_block = tid >> 6;
  unsigned out_off = kOob;
  if (e_block < PB) {
    const int pq = e_block * 16 + l16;
    if (pq < n_pixels)
      out_off = static_cast<unsigned>((pixel0 + pq) * g.features + f0 + 4 * q) *
                4u;
  }
  __syncthreads();  // every wave is done with its tile buffer
#pragma unroll
  for (int i = 0; i < FA; ++i) {
#pragma unroll
    for (int j = 0; j < PB; ++j) part[(wave * PB + j) * 64 + lane] = acc[i][j];
    __syncthreads();
    if (e_block < PB) {
      float4v sum = part[e_block * 64 + lane];
#pragma unroll
      for (int w = 1; w < kWaves; ++w)
        sum += part[(w * PB + e_block) * 64 + lane];
      if (bias != nullptr) {
        const float* b = bias + f0 + 16 * i + 4 * q;
        sum += float4v{b[0], b[1], b[2], b[3]};
      }
      if (relu) {
#pragma unroll
        for (int v = 0; v < 4; ++v) sum[v] = fmaxf(sum[v], 0.f);
      }
      __builtin_amdgcn_raw_buffer_store_b128(
          __builtin_bit_cast(uint4v, sum), dst_rsrc,
          out_off == kOob ? kOob : out_off + static_cast<unsigned>(64 * i), 0,
          0);
    }
    __syncthreads();
  }
}

struct SplitPlan {
  SplitTile g;
  int fa = 0, pb = 0;
  size_t lds_bytes = 0;  // 0: shape not supported
  long cost = 0;         // blocks a wave holds x rounds over the compute units
  unsigned n_groups = 0;
};

SplitPlan plan_tile(const snn_hip_conv2d_params& p, int fa, int pb,
                    int tile_pixels) {
  SplitPlan plan;
  SplitTile& g = plan.g;
  g.batch = p.batch; g.in_rows = p.in_rows; g.in_cols = p.in_cols;
  g.channels = p.channels; g.features = p.features;
  g.out_rows = p.out_rows; g.out_cols = p.out_cols;
  g.win_rows = p.window_rows; g.win_cols = p.window_cols;
  g.pad_rows = p.pad_rows; g.pad_cols = p.pad_cols;
  g.total_pixels = p.batch * p.out_rows * p.out_cols;
  g.tile_pixels = tile_pixels;
  g.padded_rows = p.out_rows + p.window_rows - 1;
  g.halo_cols = p.out_cols + p.window_cols - 1;
  // Padded rows a tile spans, the largest over all tiles (their position
  // inside an image repeats every image / gcd tiles).
  const long image = static_cast<long>(p.out_rows) * p.out_cols;
  const long n_tiles = ceil_div(g.total_pixels, tile_pixels);
  const long period = std::min<long>(
      n_tiles, image / std::gcd<long>(image, tile_pixels) + 1);
  auto padded_row = [&](long pixel) {
    const long row = pixel / p.out_cols;
    return row / p.out_rows * g.padded_rows + row % p.out_rows;
  };
  long lds_rows = 0;
  for (long t = 0; t < period; ++t) {
    const long first = t * tile_pixels;
    const long last =
        std::min<long>(first + tile_pixels, g.total_pixels) - 1;
    lds_rows = std::max(lds_rows, padded_row(last) - padded_row(first) +
                                      p.window_rows);
  }
  g.n_slots = static_cast<int>(lds_rows) * g.halo_cols;
  g.n_fslices = p.features / (16 * fa);
  const size_t n_blocks =
      ceil_div(static_cast<size_t>(g.n_slots) * kSlotBytes, size_t{1024});
  const size_t n_table = n_blocks * 1024 / kSlotBytes + 1;
  const size_t work = std::max(kWaves * n_blocks * 1024,
                               static_cast<size_t>(kWaves) * pb * 1024);
  const size_t lds_bytes = work + n_table * 4;
  if (lds_bytes > kMaxLdsBytes || n_blocks > kMaxBlocks) return plan;
  plan.fa = fa;
  plan.pb = pb;
  plan.lds_bytes = lds_bytes;
  plan.n_groups = static_cast<unsigned>(n_tiles) *
                  static_cast<unsigned>(g.n_fslices);
  plan.cost = static_cast<long>(ceil_div(plan.n_groups,
                                         unsigned{kComputeUnits})) * fa * pb;
  return plan;
}

// Wave shapes built: 4 x 7 and 2 x 7 blocks (112 / 56 accumulator registers).
// Tiles of a whole number of rows or the work-group's capacity; the cheapest
// plan wins, ties go to the longer tile and then to more features per wave.
SplitPlan compute_plan(const snn_hip_conv2d_params& p) {
  const int total = p.batch * p.out_rows * p.out_cols;
  SplitPlan best;
  constexpr int kPb = 7;
  for (int fa : {4, 2}) {
    if (p.features % (16 * fa) != 0) continue;
    const int capacity = std::min(kPb * 16, total);
    auto consider = [&](int tile_pixels) {
      const SplitPlan plan = plan_tile(p, fa, kPb, tile_pixels);
      if (plan.lds_bytes == 0) return;
      if (best.lds_bytes == 0 || plan.cost < best.cost ||
          (plan.cost == best.cost &&
           plan.g.tile_pixels > best.g.tile_pixels))
        best = plan;
    };
    consider(capacity);
    for (int rows = capacity / p.out_cols; rows >= 1; --rows)
      consider(rows * p.out_cols);
  }
  return best;
}

SplitPlan make_plan(const snn_hip_conv2d_params& p) {
  thread_local snn_hip_conv2d_params cached_params;
  thread_local SplitPlan cached_plan;
  thread_local bool cached = false;
  if (!cached || std::memcmp(&cached_params, &p, sizeof(p)) != 0) {
    cached_plan = compute_plan(p);
    cached_params = p;
    cached = true;
  }
  return cached_plan;
}

template <int FA, int PB, bool TRANSPOSED>
void launch_plan(const float* input, const float* filter, float* output,
                 const snn_hip_conv2d_params& p, const SplitPlan& plan,
                 const float* bias, int relu, hipStream_t stream) {
  auto kernel = conv_rowsplit_f32_kernel<FA, PB, TRANSPOSED>;
  static const hipError_t attr = hipFuncSetAttribute(
      reinterpret_cast<const void*>(kernel),
      hipFuncAttributeMaxDynamicSharedMemorySize, kMaxLdsBytes);
  (void)attr;
  const size_t x = static_cast<size_t>(p.batch) * p.in_rows * p.in_cols *
                   p.channels;
  const size_t w = static_cast<size_t>(p.window_rows) * p.window_cols *
                   p.channels * p.features;
  const size_t y = static_cast<size_t>(p.batch) * p.out_rows * p.out_cols *
                   p.features;
  // one work-group per compute unit is what the plan's cost assumes: ask for
  // more than half of the LDS so that the dispatcher does not pair them up
  const size_t lds_bytes = std::max(plan.lds_bytes, kMaxLdsBytes / 2 + 1024);
  KernelTimer timer(stream);
  hipLaunchKernelGGL(kernel, dim3(plan.n_groups), dim3(64 * kWaves), lds_bytes,
                     stream, input, filter, output, plan.g,
                     static_cast<unsigned>(x * 4), static_cast<unsigned>(w * 4),
                     static_cast<unsigned>(y * 4), plan.n_groups, bias, relu);
}

}  // namespace

// `p` describes the convolution the kernel runs (for an input gradient: the
// forward convolution over dY).
bool conv2d_rowsplit_supports(const snn_hip_conv2d_params& p) {
  const size_t x = static_cast<size_t>(p.batch) * p.in_rows * p.in_cols *
                   p.channels;
  const size_t y = static_cast<size_t>(p.batch) * p.out_rows * p.out_cols *
                   p.features;
  const size_t w = static_cast<size_t>(p.window_rows) * p.window_cols *
                   p.channels * p.features;
  if (p.stride_rows != 1 || p.stride_cols != 1) return false;
  if (p.channels % (kKC * kWaves) != 0 || p.features % 32 != 0) return false;
  // 1x1 windows: only long reductions (at 512 channels a wave has four
  // channel blocks and the general kernels measured faster, at 1024 this one
  // is 15 % ahead)
  if (p.window_rows * p.window_cols == 1) {
    int min_channels = 1024;
    if (const char* tune = SNN_TUNING_ENV("SNN_HIP_ROWSPLIT_1X1"))
      min_channels = std::atoi(tune);
    if (p.channels < min_channels) return false;
  }
  if (std::max(std::max(x, y), w) * 4 > kMaxBufferBytes) return false;
  const SplitPlan plan = make_plan(p);
  if (plan.lds_bytes == 0) return false;
  // most compute units busy, most block slots real output
  const double blocks = static_cast<double>(plan.g.total_pixels) / 16.0 *
                        (p.features / 16);
  const double slots = static_cast<double>(plan.cost) * kComputeUnits;
  return plan.n_groups >= 200 && blocks >= 0.8 * slots;
}

int launch_conv2d_rowsplit_f32(const float* input, const float* filter,
                               float* output, const snn_hip_conv2d_params& p,
                               hipStream_t stream, bool transposed_filter,
                               const LaunchOptions* epilogue) {
  const SplitPlan plan = make_plan(p);
  if (plan.lds_bytes == 0) return SNN_HIP_INVALID_ALGORITHM;
  static const bool print_plan =
      SNN_TUNING_ENV("SNN_HIP_ROWTILE_PLAN") != nullptr;
  if (print_plan)
    fprintf(stderr,
            "rowsplit f32: %d x %d blocks per wave, %d pixels/tile, %u "
            "work-groups, %zu B LDS\n",
            plan.fa, plan.pb, plan.g.tile_pixels, plan.n_groups,
            plan.lds_bytes);
  const bool fold = epilogue != nullptr && epilogue->wanted();
  const float* bias = fold ? epilogue->bias : nullptr;
  const int relu = fold && epilogue->relu ? 1 : 0;
#define SNN_ROWSPLIT(FA)                                                      \
  if (plan.fa == FA) {                                                        \
    if (transposed_filter)                                                    \
      launch_plan<FA, 7, true>(input, filter, output, p, plan, bias, relu,    \
                               stream);                                       \
    else                                                                      \
      launch_plan<FA, 7, false>(input, filter, output, p, plan, bias, relu,   \
                                stream);                                      \
  }
  SNN_ROWSPLIT(4)
  SNN_ROWSPLIT(2)
#undef SNN_ROWSPLIT
  const hipError_t err = hipGetLastError();
  if (err != hipSuccess)
    return report_hip_error(err, "conv_rowsplit_f32_kernel");
  if (fold && epilogue->applied != nullptr) *epilogue->applied = true;
  return SNN_HIP_OK;
}

}  // namespace snn
