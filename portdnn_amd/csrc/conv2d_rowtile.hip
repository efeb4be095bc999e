// fp32 stride-1 convolution on MFMA (gfx950) with the input tile resident in
// LDS: the kernel behind the Tiled and Im2col tags for windows larger than
// 1x1 (forward, and the stride-1 input gradient run as a forward convolution
// over dY with mirrored taps).  portDNN's counterparts are the tiled kernel
// (src/conv2d/tiled/kernels.h:99-190) and im2col's tile extraction followed by
// a matmul (src/conv2d/im2col/kernels/extract_input_tiles.h); both produce
// out[n][y][x][k] = sum_{r,s,c} in[n][y+r-pad][x+s-pad][c] * w[r][s][c][k].
//
// The implicit-GEMM kernel in conv2d_igemm.hip gathers every input pixel once
// per filter tap through the vector-memory pipeline, and that gather, not the
// matrix pipe, bounds it.  Here a work-group of eight waves owns a run of
// consecutive output pixels (images, rows and columns flattened, so a tile may
// start inside a row and run over an image boundary) and 64 features:
//
//   * the input rows those pixels need, halo and zero padding included, are
//     loaded into LDS once per block of 16 channels, [pixel slot][16 floats +
//     16 bytes of padding], by buffer loads that write LDS directly (out of
//     range offsets write the zeros of the padding); every filter tap reads
//     the same tile at a slot offset of r * Wh + s.  Two tiles alternate: the
//     next channel block loads while the current one is multiplied;
//   * the filter never touches LDS and is not re-packed: with features as the
//     rows of v_mfma_f32_16x16x4_f32, lane (f = l % 16, q = l / 16) needs
//     w[tap][c0 + 4 q + t][f0 + f] for the four instructions t = 0..3 of a
//     16-channel step, four 4-byte loads from the HWCF tensor (one 16-byte
//     load for the input gradient, whose reduction index is contiguous), all
//     L2 hits, six fragment buffers in rotation, five steps ahead;
//   * the pixel operand of those four instructions is one ds_read_b128 of
//     channels c0 + 4 q .. + 3 of the lane's pixel slot (l % 16); a slot is
//     five 16-byte pieces, so 16 consecutive slots fall into different banks;
//   * wave (wf, wp) owns feature block wf (16 features) and PB pixel blocks of
//     16: per step it issues 4 (or 1) filter loads and PB LDS reads for 4 PB
//     matrix instructions, which leaves the loop bound by the matrix pipe;
//   * a lane ends with four consecutive features of a pixel: one 16-byte
//     store per block, bias and ReLU applied on the way when asked for.
//
// The tile length is chosen on the host so that the work-groups come out as
// a whole number of rounds over the 256 compute units with as few idle pixel
// blocks as possible (batch-32 ResNet: 392 pixels x 64 features for 56x56x64,
// 196 for 28x28x128: one work-group per compute unit each; the deeper layers
// have too few pixels for this shape and run on conv2d_rowsplit.hip).
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
constexpr int kKC = 16;                 // channels per LDS tile
constexpr int kSlotBytes = kKC * 4 + 16;  // one pad piece: 5 pieces per slot
constexpr int kWaves = 8;               // 4 feature blocks x 2 pixel groups
constexpr int kFeatures = 64;           // features per work-group
constexpr int kComputeUnits = 256;

struct RowTile {
  int batch, in_rows, in_cols, channels, features;
  int out_rows, out_cols;
  int win_rows, win_cols, pad_rows, pad_cols;
  int tile_pixels;   // output pixels (flattened n, y, x) per work-group
  int total_pixels;  // batch * out_rows * out_cols
  int padded_rows;   // Hp = out_rows + win_rows - 1: padded rows per image
  int halo_cols;     // Wh = out_cols + win_cols - 1
  int n_slots;       // LDS pixel slots per tile = lds rows * Wh
  int n_fslices;     // features / 64
};

__device__ inline __amdgpu_buffer_rsrc_t make_rsrc(const void* p,
                                                   unsigned bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, bytes,
                                           0x00020000);
}

// Position of a reduction step: filter tap (r, c) of channel block `chunk`.
struct StepPos {
  int r = 0, c = 0, chunk = 0;
};

// PB: pixel blocks of 16 per wave.  MULTI: more than one channel block.
// WIN3: 3x3 window, whose reduction loop is unrolled over a filter row.
// TRANSPOSED: the filter operand is w[taps - 1 - tap][f][c] of an HWCF tensor
// whose channel count is this launch's feature count (the input gradient).
template <int PB, bool MULTI, bool WIN3, bool TRANSPOSED>
__global__ void __launch_bounds__(64 * kWaves)
    conv_rowtile_f32_kernel(const float* __restrict__ src,
                            const float* __restrict__ wgt,
                            float* __restrict__ dst, RowTile g,
                            unsigned src_bytes, unsigned wgt_bytes,
                            unsigned dst_bytes, unsigned n_groups,
                            const float* __restrict__ bias, int relu) {
  constexpr int NT = 64 * kWaves;
  extern __shared__ __align__(16) unsigned char lds[];
  typedef __attribute__((address_space(3))) void* lds_ptr;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wf = wave & 3, wp = wave >> 2;
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
  unsigned char* const bufs = lds;
  unsigned* const table =
      reinterpret_cast<unsigned*>(lds + (MULTI ? 2 : 1) * buf_bytes);

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

  // Starts the loads of one channel block into an LDS tile: wave w takes the
  // 1 KB blocks w, w + 8, ...; lane l fills bytes 16 l .. 16 l + 15 of its
  // block, which belong to piece (position % slot bytes) / 16 of slot
  // position / slot bytes; the pad piece of a slot loads from out of range
  // (zeros), and so do padding pixels: the vector offset is the one the
  // hardware range-checks, so the channel block's offset is added to it.
  auto start_tile = [&](unsigned char* buf, int chunk) {
    const unsigned coff = static_cast<unsigned>(chunk) * (kKC * 4u);
    for (int block = wave; block < n_blocks; block += kWaves) {
      const int pos = block * 1024 + lane * 16;
      const int slot = pos / kSlotBytes;
      const int piece = (pos - slot * kSlotBytes) >> 4;
      const unsigned base = table[slot];
      const unsigned voff =
          (piece < kKC / 4 && base != kOob)
              ? base + coff + static_cast<unsigned>(piece) * 16u
              : kOob;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(
          src_rsrc, (lds_ptr)(buf + block * 1024), 16, voff, 0, 0, 0);
    }
  };
  start_tile(bufs, 0);

  // LDS byte offset (tap (0,0), channel 4 q of the block) of this lane's
  // pixel in each of its pixel blocks, and the flattened output pixel (-1:
  // none; such lanes multiply slot 0 and store nothing).
  const int l16 = lane & 15;
  const int q = lane >> 4;
  int lane_base[PB];
  int out_pixel[PB];
#pragma unroll
  for (int j = 0; j < PB; ++j) {
    const int pq = (wp * PB + j) * 16 + l16;
    lane_base[j] = q * 16;
    out_pixel[j] = -1;
    if (pq < n_pixels) {
      const int m = pixel0 + pq;
      const int orow = m / g.out_cols;
      const int x = m - orow * g.out_cols;
      const int n = orow / g.out_rows;
      const int lrow = n * g.padded_rows + (orow - n * g.out_rows) -
                       first_padded;
      lane_base[j] = (lrow * g.halo_cols + x) * kSlotBytes + q * 16;
      out_pixel[j] = m;
    }
  }

  const int taps = g.win_rows * g.win_cols;
  const int n_chunks = g.channels / kKC;
  const int f_lane = fslice * kFeatures + wf * 16 + l16;
  // Filter operand of a step.  Forward: w[tap][chunk * 16 + 4 q + t][f_lane],
  // four loads a row of the filter apart.  Input gradient: w[taps - 1 - tap]
  // [f_lane][chunk * 16 + 4 q .. + 3], one load.  The lane's part of the
  // address never changes; the step's part is wave-uniform and travels in the
  // scalar offset, so a load costs no vector arithmetic.  The prefetch runs
  // ahead of the last step: those loads read the start of the filter.
  const unsigned a_lane =
      TRANSPOSED
          ? static_cast<unsigned>(f_lane * g.channels + 4 * q) * 4u
          : static_cast<unsigned>(4 * q * g.features + f_lane) * 4u;
  const unsigned a_row = static_cast<unsigned>(g.features) * 4u;
  auto load_a = [&](float4v& frag, const StepPos& s) {
    const int tap = s.r * g.win_cols + s.c;
    const bool ok = s.chunk < n_chunks;
    if (TRANSPOSED) {
      const unsigned soff =
          ok ? static_cast<unsigned>((taps - 1 - tap) * g.features *
                                         g.channels +
                                     s.chunk * kKC) * 4u
             : 0u;
      frag = __builtin_bit_cast(
          float4v,
          __builtin_amdgcn_raw_buffer_load_b128(wgt_rsrc, a_lane, soff, 0));
    } else {
      const unsigned soff =
          ok ? static_cast<unsigned>(tap * g.channels + s.chunk * kKC) * a_row
             : 0u;
#pragma unroll
      for (int t = 0; t < 4; ++t)
        frag[t] = __builtin_bit_cast(
            float, __builtin_amdgcn_raw_buffer_load_b32(
                       wgt_rsrc, a_lane,
                       soff + static_cast<unsigned>(t) * a_row, 0));
    }
  };
  auto advance = [&](StepPos& s) {
    const int row_ends = ++s.c == g.win_cols ? 1 : 0;
    s.c = row_ends ? 0 : s.c;
    s.r += row_ends;
    const int chunk_ends = s.r == g.win_rows ? 1 : 0;
    s.r = chunk_ends ? 0 : s.r;
    s.chunk += chunk_ends;
  };

  // Filter fragments: six buffers in rotation, a load has five steps of
  // matrix instructions to arrive.  Vector-memory loads complete in order, so
  // a filter load issued behind the loads of the next tile waits for them:
  // the distance has to cover the latency of a tile load from HBM.
  constexpr int kDepth = 6;
  float4v a_buf[kDepth];
  StepPos a_pos;
#pragma unroll
  for (int d = 0; d + 1 < kDepth; ++d) {
    load_a(a_buf[d], a_pos);
    advance(a_pos);
  }

  float4v acc[PB];
#pragma unroll
  for (int j = 0; j < PB; ++j) acc[j] = float4v{0.f, 0.f, 0.f, 0.f};

  // The first tile has landed once no vector-memory load is outstanding.
  __builtin_amdgcn_s_waitcnt(0x0F70);
  __syncthreads();
  if (MULTI && n_chunks > 1) start_tile(bufs + buf_bytes, 1);

  int cur_off = 0;  // byte offset of the tile being multiplied
  // Pixel operands: two sets, the one of the next step is read from LDS
  // while the matrix instructions of the current one run.
  float4v b_buf[2][PB];
  auto mfma_step = [&](const float4v& a, const float4v (&b)[PB]) {
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int j = 0; j < PB; ++j)
        acc[j] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[t], b[j][t], acc[j], 0,
                                                      0, 0);
    __builtin_amdgcn_sched_barrier(0);
  };
  // End of a channel block (not the last).  The loads into the next tile
  // were issued at the block's start, before the filter loads of all of its
  // steps; vector-memory loads complete in order, so they have landed once at
  // most the filter loads of the last kDepth - 1 steps are outstanding (or,
  // for windows with fewer taps than that, none).  No fence: the pixel
  // operands of this tile have all been consumed, and the barrier alone makes
  // every wave's part of the next tile visible.  The tile just finished is
  // then free for the block after next.
  auto next_tile = [&](int next_chunk) {
    constexpr int kLoadsPerStep = TRANSPOSED ? 1 : 4;
    constexpr int kInFlight = (kDepth - 1) * kLoadsPerStep;
    if (taps >= kDepth - 1)
      __builtin_amdgcn_s_waitcnt(0x0F70 | (kInFlight & 15) |
                                 ((kInFlight >> 4) << 14));
    else
      __builtin_amdgcn_s_waitcnt(0x0F70);
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
    const int done_off = cur_off;
    cur_off = buf_bytes - cur_off;
    if (next_chunk + 1 < n_chunks) start_tile(bufs + done_off, next_chunk + 1);
  };

  if constexpr (WIN3) {
    // 3x3 window: the loop runs over filter rows with the three taps of a row
    // unrolled.  A lane keeps the LDS address of the row's first tap for each
    // of its pixel blocks; the taps of the row are compile-time offsets from
    // it, so pixel operands cost vector arithmetic once a row, not once a
    // step.  A row takes three filter buffers and flips the operand sets, so
    // rows alternate between two register assignments.
    int rb[PB];
#pragma unroll
    for (int j = 0; j < PB; ++j) rb[j] = lane_base[j];
    const int row_step = g.halo_cols * kSlotBytes;
    auto read_row = [&](float4v (&b)[PB], const int (&base)[PB], int tap_col) {
#pragma unroll
      for (int j = 0; j < PB; ++j)
        b[j] = *reinterpret_cast<const float4v*>(bufs + base[j] +
                                                 tap_col * kSlotBytes);
    };
    read_row(b_buf[0], rb, 0);
    int r = 0, chunk = 0;
    auto do_row = [&](const float4v& a0, const float4v& a1, const float4v& a2,
                      float4v& f0, float4v& f1, float4v& f2,
                      float4v (&bx)[PB], float4v (&by)[PB]) {
      load_a(f0, a_pos);
      advance(a_pos);
      read_row(by, rb, 1);
      mfma_step(a0, bx);
      load_a(f1, a_pos);
      advance(a_pos);
      read_row(bx, rb, 2);
      mfma_step(a1, by);
      load_a(f2, a_pos);
      advance(a_pos);
      // the next filter row (after the last one the tiles swap and the
      // operands are read again behind the barrier; this read then only
      // keeps the instruction stream uniform)
      const bool chunk_ends = r == 2;
      const int to_next_row = chunk_ends ? -2 * row_step : row_step;
#pragma unroll
      for (int j = 0; j < PB; ++j) rb[j] += to_next_row;
      read_row(by, rb, 0);
      mfma_step(a2, bx);
      r = chunk_ends ? 0 : r + 1;
      if (chunk_ends) {
        ++chunk;
        if (MULTI && chunk < n_chunks) {
          const int old_off = cur_off;
          next_tile(chunk);
          const int to_next_tile = cur_off - old_off;
#pragma unroll
          for (int j = 0; j < PB; ++j) rb[j] += to_next_tile;
          read_row(by, rb, 0);
        }
      }
    };
    const int total_rows = 3 * n_chunks;
    int row = 0;
    for (; row + 2 <= total_rows; row += 2) {
      do_row(a_buf[0], a_buf[1], a_buf[2], a_buf[5], a_buf[0], a_buf[1],
             b_buf[0], b_buf[1]);
      do_row(a_buf[3], a_buf[4], a_buf[5], a_buf[2], a_buf[3], a_buf[4],
             b_buf[1], b_buf[0]);
    }
    if (row < total_rows)
      do_row(a_buf[0], a_buf[1], a_buf[2], a_buf[5], a_buf[0], a_buf[1],
             b_buf[0], b_buf[1]);
  } else {
    auto read_b = [&](float4v (&b)[PB], int offset) {
#pragma unroll
      for (int j = 0; j < PB; ++j)
        b[j] = *reinterpret_cast<const float4v*>(bufs + lane_base[j] + offset);
    };
    read_b(b_buf[0], 0);
    StepPos b_pos;  // the step being multiplied
    auto do_step = [&](const float4v& a_use, float4v& a_fill,
                       const float4v (&b_use)[PB], float4v (&b_fill)[PB]) {
      const int chunk = b_pos.chunk;
      advance(b_pos);
      const bool chunk_ends = b_pos.chunk != chunk;
      load_a(a_fill, a_pos);
      advance(a_pos);
      // (after a channel block's last step the operands are read again behind
      // the barrier; this read then only keeps the instruction stream uniform)
      read_b(b_fill,
             cur_off + (chunk_ends ? 0
                                   : (b_pos.r * g.halo_cols + b_pos.c) *
                                         kSlotBytes));
      mfma_step(a_use, b_use);
      if (MULTI && chunk_ends && b_pos.chunk < n_chunks) {
        next_tile(b_pos.chunk);
        read_b(b_fill, cur_off);
      }
    };
    // Six steps a turn: the filter buffers and the two operand sets are then
    // the same registers in every turn.
    const int total_steps = n_chunks * taps;
    int done = 0;
    for (; done + 6 <= total_steps; done += 6) {
      do_step(a_buf[0], a_buf[5], b_buf[0], b_buf[1]);
      do_step(a_buf[1], a_buf[0], b_buf[1], b_buf[0]);
      do_step(a_buf[2], a_buf[1], b_buf[0], b_buf[1]);
      do_step(a_buf[3], a_buf[2], b_buf[1], b_buf[0]);
      do_step(a_buf[4], a_buf[3], b_buf[0], b_buf[1]);
      do_step(a_buf[5], a_buf[4], b_buf[1], b_buf[0]);
    }
    if (done + 0 < total_steps) do_step(a_buf[0], a_buf[5], b_buf[0], b_buf[1]);
    if (done + 1 < total_steps) do_step(a_buf[1], a_buf[0], b_buf[1], b_buf[0]);
    if (done + 2 < total_steps) do_step(a_buf[2], a_buf[1], b_buf[0], b_buf[1]);
    if (done + 3 < total_steps) do_step(a_buf[3], a_buf[2], b_buf[1], b_buf[0]);
    if (done + 4 < total_steps) do_step(a_buf[4], a_buf[3], b_buf[0], b_buf[1]);
  }
  // every wave's tile loads have landed before the work-group ends
  __builtin_amdgcn_s_waitcnt(0x0F70);

  // acc[j][i] is feature f0 + 4 q + i of pixel l16 of block j.
  const __amdgpu_buffer_rsrc_t dst_rsrc = make_rsrc(dst, dst_bytes);
  const int f_out = fslice * kFeatures + wf * 16 + 4 * q;
  float4v add = float4v{0.f, 0.f, 0.f, 0.f};
  if (bias != nullptr) {
#pragma unroll
    for (int i = 0; i < 4; ++i) add[i] = bias[f_out + i];
  }
#pragma unroll
  for (int j = 0; j < PB; ++j) {
    float4v v = acc[j] + add;
    if (relu) {
#pragma unroll
      for (int i = 0; i < 4; ++i) v[i] = fmaxf(v[i], 0.f);
    }
    const unsigned off =
        out_pixel[j] >= 0
            ? static_cast<unsigned>(out_pixel[j] * g.features + f_out) * 4u
            : kOob;
    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(uint4v, v),
                                           dst_rsrc, off, 0, 0);
  }
}

struct RowTilePlan {
  RowTile g;
  int pb = 0;            // pixel blocks of 16 per wave
  size_t lds_bytes = 0;  // 0: shape not supported
  long cost = 0;
  unsigned n_groups = 0;
};

// Geometry for work-groups of `tile_pixels` consecutive output pixels;
// lds_bytes == 0 when the tile does not fit.  The cost counts matrix
// instruction slots per SIMD: rounds of work-groups over the compute units
// times the pixel blocks of a wave.
RowTilePlan plan_tile(const snn_hip_conv2d_params& p, int pb,
                      int tile_pixels) {
  RowTilePlan plan;
  RowTile& g = plan.g;
  g.batch = p.batch; g.in_rows = p.in_rows; g.in_cols = p.in_cols;
  g.channels = p.channels; g.features = p.features;
  g.out_rows = p.out_rows; g.out_cols = p.out_cols;
  g.win_rows = p.window_rows; g.win_cols = p.window_cols;
  g.pad_rows = p.pad_rows; g.pad_cols = p.pad_cols;
  g.total_pixels = p.batch * p.out_rows * p.out_cols;
  g.tile_pixels = tile_pixels;
  g.padded_rows = p.out_rows + p.window_rows - 1;
  g.halo_cols = p.out_cols + p.window_cols - 1;
  // Padded rows a tile spans: from the padded row of its first pixel to the
  // padded row of its last pixel plus the window, the largest over all tiles
  // (their position inside an image repeats every image / gcd tiles).
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
  g.n_fslices = p.features / kFeatures;
  const int n_chunks = p.channels / kKC;
  const size_t n_blocks =
      ceil_div(static_cast<size_t>(g.n_slots) * kSlotBytes, size_t{1024});
  const size_t n_table = n_blocks * 1024 / kSlotBytes + 1;
  const size_t lds_bytes =
      (n_chunks > 1 ? 2 : 1) * n_blocks * 1024 + n_table * 4;
  if (lds_bytes > kMaxLdsBytes) return plan;
  plan.pb = pb;
  plan.lds_bytes = lds_bytes;
  plan.n_groups = static_cast<unsigned>(n_tiles) *
                  static_cast<unsigned>(g.n_fslices);
  plan.cost = static_cast<long>(ceil_div(plan.n_groups,
                                         unsigned{kComputeUnits})) * pb;
  return plan;
}

// Wave shapes: smaller ones measured slower than the implicit-GEMM kernel
// (too few matrix instructions per filter load and per barrier).
constexpr int kPixelBlocks[] = {7, 10, 13};

// Tile sizes tried for every wave shape: the full capacity of the work-group
// (tiles then start anywhere in a row) and every whole number of rows below
// it that still needs this wave shape.  Cheapest first; ties go to the longer
// tile (less halo per pixel).
RowTilePlan compute_plan(const snn_hip_conv2d_params& p) {
  const int total = p.batch * p.out_rows * p.out_cols;
  RowTilePlan best;
  int below = 0;  // capacity of the next smaller wave shape
  for (int pb : kPixelBlocks) {
    const int capacity = std::min(2 * pb * 16, total);
    auto consider = [&](int tile_pixels) {
      const RowTilePlan plan = plan_tile(p, pb, tile_pixels);
      if (plan.lds_bytes == 0) return;
      if (best.lds_bytes == 0 || plan.cost < best.cost ||
          (plan.cost == best.cost &&
           plan.g.tile_pixels > best.g.tile_pixels))
        best = plan;
    };
    consider(capacity);
    for (int rows = capacity / p.out_cols; rows >= 1; --rows) {
      if (rows * p.out_cols <= below) break;
      consider(rows * p.out_cols);
    }
    below = capacity;
    if (capacity == total) break;
  }
  return best;
}

// The plan of the most recent shape is kept per thread: layers are usually
// launched many times with the same parameters.
RowTilePlan make_plan(const snn_hip_conv2d_params& p) {
  thread_local snn_hip_conv2d_params cached_params;
  thread_local RowTilePlan cached_plan;
  thread_local bool cached = false;
  if (!cached || std::memcmp(&cached_params, &p, sizeof(p)) != 0) {
    cached_plan = compute_plan(p);
    cached_params = p;
    cached = true;
  }
  return cached_plan;
}

template <int PB, bool MULTI, bool WIN3, bool TRANSPOSED>
void launch_plan(const float* input, const float* filter, float* output,
                 const snn_hip_conv2d_params& p, const RowTilePlan& plan,
                 const float* bias, int relu, hipStream_t stream) {
  auto kernel = conv_rowtile_f32_kernel<PB, MULTI, WIN3, TRANSPOSED>;
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
  // A compute unit can hold two work-groups of the smaller wave shapes, and
  // the dispatcher then fills some units twice while others stay empty.  When
  // there is at most one work-group per compute unit anyway, asking for more
  // than half of the LDS keeps them apart.
  const size_t lds_bytes =
      plan.n_groups <= kComputeUnits
          ? std::max(plan.lds_bytes, kMaxLdsBytes / 2 + 1024)
          : plan.lds_bytes;
  KernelTimer timer(stream);
  hipLaunchKernelGGL(kernel, dim3(plan.n_groups), dim3(64 * kWaves),
                     lds_bytes, stream, input, filter, output, plan.g,
                     static_cast<unsigned>(x * 4), static_cast<unsigned>(w * 4),
                     static_cast<unsigned>(y * 4), plan.n_groups, bias, relu);
}

template <int PB, bool MULTI, bool WIN3>
void launch_direction(const float* input, const float* filter, float* output,
                      const snn_hip_conv2d_params& p, const RowTilePlan& plan,
                      bool transposed, const float* bias, int relu,
                      hipStream_t stream) {
  if (transposed)
    launch_plan<PB, MULTI, WIN3, true>(input, filter, output, p, plan, bias,
                                       relu, stream);
  else
    launch_plan<PB, MULTI, WIN3, false>(input, filter, output, p, plan, bias,
                                        relu, stream);
}

template <int PB>
bool launch_shape(const float* input, const float* filter, float* output,
                  const snn_hip_conv2d_params& p, const RowTilePlan& plan,
                  bool transposed, const float* bias, int relu,
                  hipStream_t stream) {
  if (plan.pb != PB) return false;
  const bool multi = p.channels > kKC;
  const bool win3 = p.window_rows == 3 && p.window_cols == 3;
  if (multi && win3)
    launch_direction<PB, true, true>(input, filter, output, p, plan,
                                     transposed, bias, relu, stream);
  else if (multi)
    launch_direction<PB, true, false>(input, filter, output, p, plan,
                                      transposed, bias, relu, stream);
  else if (win3)
    launch_direction<PB, false, true>(input, filter, output, p, plan,
                                      transposed, bias, relu, stream);
  else
    launch_direction<PB, false, false>(input, filter, output, p, plan,
                                       transposed, bias, relu, stream);
  return true;
}

}  // namespace

// `p` describes the convolution the kernel runs (for an input gradient: the
// forward convolution over dY, see launch_conv2d_rowtile_f32).
bool conv2d_rowtile_supports(const snn_hip_conv2d_params& p) {
  const size_t x = static_cast<size_t>(p.batch) * p.in_rows * p.in_cols *
                   p.channels;
  const size_t y = static_cast<size_t>(p.batch) * p.out_rows * p.out_cols *
                   p.features;
  const size_t w = static_cast<size_t>(p.window_rows) * p.window_cols *
                   p.channels * p.features;
  if (p.stride_rows != 1 || p.stride_cols != 1) return false;
  if (p.channels % kKC != 0 || p.features % kFeatures != 0) return false;
  // 1x1 windows have no taps to reuse an LDS tile over
  if (p.window_rows * p.window_cols == 1) return false;
  if (std::max(std::max(x, y), w) * 4 > kMaxBufferBytes) return false;
  const RowTilePlan plan = make_plan(p);
  if (plan.lds_bytes == 0) return false;
  // Worth it when most compute units get a work-group and most of the wave
  // tiles' 16 x 16 blocks are real output: the share of block slots (rounds x
  // compute units x 8 waves x PB) that the output fills.
  const double blocks = static_cast<double>(plan.g.total_pixels) / 16.0 *
                        (p.features / 16);
  const double slots = static_cast<double>(plan.cost) * kComputeUnits * kWaves;
  return plan.n_groups >= 200 && blocks >= 0.8 * slots;
}

int launch_conv2d_rowtile_f32(const float* input, const float* filter,
                              float* output, const snn_hip_conv2d_params& p,
                              hipStream_t stream, bool transposed_filter,
                              const LaunchOptions* epilogue) {
  const RowTilePlan plan = make_plan(p);
  if (plan.lds_bytes == 0) return SNN_HIP_INVALID_ALGORITHM;
  static const bool print_plan = SNN_TUNING_ENV("SNN_HIP_ROWTILE_PLAN") != nullptr;
  if (print_plan)
    fprintf(stderr,
            "rowtile f32: %d pixel blocks per wave, %d pixels/tile, %u "
            "work-groups, %zu B LDS\n",
            plan.pb, plan.g.tile_pixels, plan.n_groups, plan.lds_bytes);
  const bool fold = epilogue != nullptr && epilogue->wanted();
  const float* bias = fold ? epilogue->bias : nullptr;
  const int relu = fold && epilogue->relu ? 1 : 0;
  const bool launched =
      launch_shape<7>(input, filter, output, p, plan, transposed_filter, bias,
                      relu, stream) ||
      launch_shape<10>(input, filter, output, p, plan, transposed_filter, bias,
                       relu, stream) ||
      launch_shape<13>(input, filter, output, p, plan, transposed_filter, bias,
                       relu, stream);
  if (!launched) return SNN_HIP_INVALID_ALGORITHM;
  const hipError_t err = hipGetLastError();
  if (err != hipSuccess)
    return report_hip_error(err, "conv_rowtile_f32_kernel");
  if (fold && epilogue->applied != nullptr) *epilogue->applied = true;
  return SNN_HIP_OK;
}

}  // namespace snn
