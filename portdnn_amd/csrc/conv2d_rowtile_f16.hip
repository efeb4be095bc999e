// Half-precision stride-1 forward convolution on MFMA (gfx950) with the
// input tile resident in LDS: binary16 operands, fp32 accumulation, binary16
// result.
//
// The implicit-GEMM kernel in conv2d_igemm_f16.hip gathers every input pixel
// once per filter tap through the vector-memory pipeline and passes both
// operands through LDS; at 32x32x16 f16 MFMA rates that makes LDS and the
// texture path the limit, not the matrix cores.  Here a work-group owns a run
// of consecutive output pixels (images, rows and columns flattened, so a tile
// may start inside a row and run over an image boundary) and a slice of the
// features:
//
//   * the input rows those outputs need (the tile plus its halo, zero padding
//     included as explicit zero pixels) are loaded into LDS once per block of
//     KC channels, [pixel slot][KC halves + 16 bytes of padding], by buffer
//     loads that write LDS directly; every filter tap then reads the same LDS
//     tile at a slot offset of r * Wh + s;
//   * the filter never touches LDS: it is pre-packed in MFMA A-operand order,
//     [k-step][feature block of 32][lane][8 halves], and streams from global
//     memory (L2-resident) straight into registers, prefetched two units of
//     16 MFMAs ahead;
//   * features are the MFMA rows and pixels the columns, with the 32 feature
//     rows permuted in the packed filter so that a lane ends up holding 16
//     consecutive features of one pixel: the epilogue is two 16-byte stores
//     per lane per 32x32 block.
//
// Each wave owns 2 feature blocks x 4 pixel blocks (64 features x 128
// pixels, 128 accumulator registers): per 16-deep reduction step it reads
// 4 KB from LDS and 2 KB of filter for 8 MFMAs.  Layers with too few such
// tiles to fill the SIMDs use 2 x 2 blocks per wave instead.
//
// portDNN's half build accumulates in half (e.g. `DataType out_val{0}` with
// T = cl::sycl::half in src/conv2d/direct/kernels_nhwc.h:92); accumulating in
// fp32 is more accurate and stays inside the 1e-2 relative bar against it.
#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <numeric>

#include "gemm_tile.h"
#include "snn_kernels.h"

namespace snn {
namespace {

using gemm::float16v;
using gemm::xcd_remap;

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef unsigned int uint4v __attribute__((ext_vector_type(4)));
constexpr unsigned kOob = 0x7FFFFFF0u;
constexpr int kStoreAux = 2;  // the output is written once: stream it (slc)
constexpr size_t kMaxBufferBytes = 0x7FFFFFF0u;
constexpr int kFA = 2;  // feature blocks (of 32) per wave
constexpr size_t kMaxLdsBytes = 160 * 1024;

struct RowTile {
  int batch, in_rows, in_cols, channels, features;
  int out_rows, out_cols;
  int win_rows, win_cols, pad_rows, pad_cols;
  int tile_pixels;   // output pixels (flattened n, y, x) per work-group
  int total_pixels;  // batch * out_rows * out_cols
  int padded_rows;  // Hp = out_rows + win_rows - 1: padded input rows per image
  int halo_cols;    // Wh = out_cols + win_cols - 1
  int n_slots;      // LDS pixel slots per tile = lds rows * Wh
  int n_fslices;    // features / (64 * WF)
};

__device__ inline __amdgpu_buffer_rsrc_t make_rsrc(const void* p,
                                                   unsigned bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, bytes,
                                           0x00020000);
}

// wpk[step][fb][lane][e] = w[tap][c][f] with step = (chunk * taps + tap) *
// (KC / 16) + ks, c = chunk * KC + ks * 16 + 8 * (lane / 32) + e and, for
// MFMA row rho = lane % 32, f = fb * 32 + 16 * ((rho / 4) % 2) + 4 * (rho / 8)
// + rho % 4: the accumulator rows 8g + 4h + i a lane holds (h = lane / 32)
// are then features 16h + 4g + i, 16 consecutive ones.  `transposed`: the
// input gradient's filter, w[taps - 1 - tap][f][c] of the HWCF tensor of a
// convolution with `features` input channels and `channels` features
// (mirrored taps, channel and feature roles swapped).
__global__ void __launch_bounds__(256)
    pack_filter_rowtile_kernel(const _Float16* __restrict__ w,
                               _Float16* __restrict__ wpk, int channels,
                               int features, int taps, int kc, int n_lanes,
                               bool transposed) {
  // One thread per (step, fb, lane): eight channel values of one feature.
  // The 32 lanes of a half-wave read 32 permuted but adjacent features.
  const int idx = blockIdx.x * 256 + threadIdx.x;
  if (idx >= n_lanes) return;
  const int lane = idx & 63;
  int t = idx >> 6;
  const int n_fb = features / 32;
  const int fb = t % n_fb;
  const int step = t / n_fb;
  const int ks_per = kc / 16;
  const int ks = step % ks_per;
  t = step / ks_per;
  const int tap = t % taps;
  const int chunk = t / taps;
  const int c = chunk * kc + ks * 16 + 8 * (lane >> 5);
  const int rho = lane & 31;
  const int f = fb * 32 + 16 * ((rho >> 2) & 1) + 4 * (rho >> 3) + (rho & 3);
  const _Float16* src =
      transposed
          ? w + (static_cast<size_t>(taps - 1 - tap) * features + f) * channels + c
          : w + (static_cast<size_t>(tap) * channels + c) * features + f;
  const size_t stride = transposed ? 1 : static_cast<size_t>(features);
  half8 v;
#pragma unroll
  for (int e = 0; e < 8; ++e) v[e] = src[static_cast<size_t>(e) * stride];
  *reinterpret_cast<half8*>(wpk + static_cast<size_t>(idx) * 8) = v;
}

// s_waitcnt immediates that wait on the vector-memory counter only.
constexpr int kWaitVm0 = 0x0F70;
constexpr int kWaitVm4 = 0x0F74;
constexpr int kWaitVm8 = 0x0F78;

// WF x WP waves: WF feature groups of 64, WP pixel groups of PB * 32.  KC =
// channels per LDS tile.  MULTI: more than one channel block (two LDS tiles,
// the next one loading while the current one is multiplied).  WIN3: 3x3
// window, whose reduction loop is unrolled over a filter row with all tap
// bookkeeping resolved at compile time.
//
// LDS tile: [pixel slot][KC halves + one 16-byte pad piece].  A slot is then
// an odd number of 16-byte pieces (5 or 9), so the ds_read_b128 of 16
// consecutive slots at the same piece touch 16 different bank groups, and a
// slot's address is linear in its index: the three taps of a filter row and
// the reduction steps of a tap are compile-time offsets of one address per
// pixel block, which leaves the reduction loop without address arithmetic.
// Tiles are filled by buffer loads that write LDS directly (64 lanes x 16
// bytes = 1 KB of consecutive LDS per instruction; the lanes that fall on pad
// pieces load from out of range), so a whole tile is in flight without
// holding registers; out-of-range offsets (padding pixels) store zeros.
template <int WF, int WP, int PB, int KC, bool MULTI, bool WIN3>
__global__ void __launch_bounds__(64 * WF * WP)
    __attribute__((amdgpu_waves_per_eu(2, 2)))
    conv_rowtile_f16_kernel(const _Float16* __restrict__ src,
                            const _Float16* __restrict__ wpk,
                            _Float16* __restrict__ dst, RowTile g,
                            unsigned src_bytes, unsigned wpk_bytes,
                            unsigned dst_bytes, unsigned n_groups) {
  constexpr int NT = 64 * WF * WP;
  constexpr int NW = WF * WP;
  constexpr int KS = KC / 16;        // MFMA reduction steps per tap
  constexpr int UPT = KS / 2;        // units of two steps per tap
  constexpr int PPS = KC / 8;        // 16-byte pieces of data per slot
  constexpr int SLOTB = KC * 2 + 16; // bytes per LDS pixel slot (one pad piece)
  extern __shared__ __align__(16) unsigned char lds[];
  typedef __attribute__((address_space(3))) void* lds_ptr;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wf = wave / WP, wp = wave % WP;
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
  const int n_blocks = (g.n_slots * SLOTB + 1023) / 1024;
  const int n_table = n_blocks * 1024 / SLOTB + 1;
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
                                   g.channels) * 2u
           : kOob;
  }
  __syncthreads();

  const __amdgpu_buffer_rsrc_t src_rsrc = make_rsrc(src, src_bytes);
  const __amdgpu_buffer_rsrc_t wpk_rsrc = make_rsrc(wpk, wpk_bytes);

  // Starts the loads of one channel block into an LDS tile: wave w takes the
  // 1 KB blocks w, w + NW, ...; lane l fills bytes 16 l .. 16 l + 15 of its
  // block, which belong to piece (position % SLOTB) / 16 of slot position /
  // SLOTB; the pad piece of a slot loads from out of range (zeros).  `soff`
  // (in range by construction) selects the channel block; padding pixels go
  // out of range through the vector offset, the only one the hardware
  // range-checks.
  auto start_tile = [&](unsigned char* buf, unsigned soff) {
    for (int block = wave; block < n_blocks; block += NW) {
      const int pos = block * 1024 + lane * 16;
      const int slot = pos / SLOTB;
      const int piece = (pos - slot * SLOTB) >> 4;
      const unsigned voff =
          piece < PPS ? table[slot] + static_cast<unsigned>(piece) * 16u : kOob;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(
          src_rsrc, (lds_ptr)(buf + block * 1024), 16, voff, soff, 0, 0);
    }
  };
  start_tile(bufs, 0);

  // LDS slot (tap (0,0)) of this lane's pixel in each of its pixel blocks,
  // and the flattened output pixel (-1: none).
  const int l32 = lane & 31;
  const int khalf = lane >> 5;
  int b_slot[PB];
  int out_pixel[PB];
#pragma unroll
  for (int j = 0; j < PB; ++j) {
    const int q = (wp * PB + j) * 32 + l32;
    b_slot[j] = 0;
    out_pixel[j] = -1;
    if (q < n_pixels) {
      const int m = pixel0 + q;
      const int orow = m / g.out_cols;
      const int x = m - orow * g.out_cols;
      const int n = orow / g.out_rows;
      const int lrow = n * g.padded_rows + (orow - n * g.out_rows) -
                       first_padded;
      b_slot[j] = lrow * g.halo_cols + x;
      out_pixel[j] = m;
    }
  }

  const int n_fb = g.features / 32;
  const int fb0 = (fslice * WF + wf) * kFA;
  const unsigned a_voff = static_cast<unsigned>(fb0 * 64 + lane) * 16u;
  const unsigned a_step_bytes = static_cast<unsigned>(n_fb) * 1024u;
  // The reduction runs in units of two MFMA steps (32 channels of one tap).
  // Filter fragments: DEPTH buffers of one unit each in rotation.  Unit u
  // multiplies out of buffer u % DEPTH while the buffer unit u - 1 used is
  // refilled with the fragments of unit u + DEPTH - 1, so a load has
  // DEPTH - 1 units of MFMAs to arrive and no register copies wait on it.
  // The smaller wave tile has half the MFMAs per unit and registers to
  // spare: it prefetches twice as far.  Reads past the end of the packed
  // filter return zeros.
  constexpr int DEPTH = (PB == 2 && !WIN3) ? 5 : 3;
  half8 a_buf[DEPTH][2][kFA];
  auto load_a = [&](half8 (&frag)[2][kFA], unsigned first_step) {
#pragma unroll
    for (int ks = 0; ks < 2; ++ks)
#pragma unroll
      for (int i = 0; i < kFA; ++i)
        frag[ks][i] = __builtin_bit_cast(
            half8, __builtin_amdgcn_raw_buffer_load_b128(
                       wpk_rsrc,
                       a_voff + static_cast<unsigned>(i) * 1024u +
                           (first_step + static_cast<unsigned>(ks)) *
                               a_step_bytes,
                       0, 0));
  };
#pragma unroll
  for (int d = 0; d + 1 < DEPTH; ++d)
    load_a(a_buf[d], static_cast<unsigned>(2 * d));

  float16v acc[kFA][PB];
#pragma unroll
  for (int i = 0; i < kFA; ++i)
#pragma unroll
    for (int j = 0; j < PB; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  // The first tile has landed once no vector-memory load is outstanding.
  __builtin_amdgcn_s_waitcnt(kWaitVm0);
  __syncthreads();

  const int taps = g.win_rows * g.win_cols;
  const int n_chunks = g.channels / KC;
  const int units_per_chunk = taps * UPT;
  const int total_units = n_chunks * units_per_chunk;
  unsigned step = 0;  // first reduction step of the unit
  half8 b_even[PB], b_odd[PB];  // pixel fragments of even / odd steps
  auto mfma_step = [&](const half8 (&a)[kFA], const half8 (&b)[PB]) {
#pragma unroll
    for (int i = 0; i < kFA; ++i)
#pragma unroll
      for (int j = 0; j < PB; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[i], b[j],
                                                           acc[i][j], 0, 0, 0);
  };
  if constexpr (WIN3) {
    // Scalar and branch instructions between MFMAs leave the matrix pipe
    // idle, so this path has none per unit: the loop runs over filter rows
    // with the three taps of a row (UPT units each) unrolled, which also
    // keeps the rotation of the three filter buffers static.
    int cur_off = 0, nxt_off = buf_bytes;
    // Byte offset inside a tile of this lane's fragment of tap (0, 0), step 0.
    // Slots are SLOTB bytes apart, so the taps of a filter row and the steps
    // of a tap are compile-time offsets from the row's address.
    int lane_base[PB];
#pragma unroll
    for (int j = 0; j < PB; ++j) lane_base[j] = b_slot[j] * SLOTB + khalf * 16;
    const int row_step = g.halo_cols * SLOTB;
    auto read_b = [&](half8 (&b)[PB], const int (&rb)[PB], int offset) {
#pragma unroll
      for (int j = 0; j < PB; ++j)
        b[j] = *reinterpret_cast<const half8*>(bufs + rb[j] + offset);
    };
    int rb[PB];  // filter row r of the current tile
#pragma unroll
    for (int j = 0; j < PB; ++j) rb[j] = cur_off + lane_base[j];
    read_b(b_even, rb, 0);
#pragma unroll 1
    for (int c = 0; c < n_chunks; ++c) {
#pragma unroll 1
      for (int r = 0; r < 3; ++r) {
        // the next filter row (after the last one the tiles swap and the
        // fragment is read again; the tile's first row will do here)
        int rb_next[PB];
#pragma unroll
        for (int j = 0; j < PB; ++j)
          rb_next[j] = r < 2 ? rb[j] + row_step : cur_off + lane_base[j];
#pragma unroll
        for (int sc = 0; sc < 3; ++sc) {
#pragma unroll
          for (int u = 0; u < UPT; ++u) {
            constexpr int kRot = 3;
            const int v = sc * UPT + u;  // unit within the filter row
            half8 (&a_use)[2][kFA] = a_buf[v % kRot];
            half8 (&a_fill)[2][kFA] = a_buf[(v + 2) % kRot];
            if constexpr (MULTI) {
              if (sc == 0 && u == 0) {
                if (r == 0 && c + 1 < n_chunks)
                  start_tile(bufs + nxt_off,
                             static_cast<unsigned>((c + 1) * KC * 2));
              }
            }
            read_b(b_odd, rb, sc * SLOTB + (2 * u + 1) * 32);
            __builtin_amdgcn_sched_barrier(0);
            // The filter prefetch issues in the shadow of the MFMAs.
            load_a(a_fill, step + 4);
            step += 2;
            mfma_step(a_use[0], b_even);
            __builtin_amdgcn_sched_barrier(0);
            if (u + 1 < UPT)
              read_b(b_even, rb, sc * SLOTB + (2 * u + 2) * 32);
            else if (sc < 2)
              read_b(b_even, rb, (sc + 1) * SLOTB);
            else
              read_b(b_even, rb_next, 0);
            __builtin_amdgcn_sched_barrier(0);
            mfma_step(a_use[1], b_odd);
            __builtin_amdgcn_sched_barrier(0);
          }
        }
#pragma unroll
        for (int j = 0; j < PB; ++j) rb[j] = rb_next[j];
      }
      if constexpr (MULTI) {
        // End of the channel block.  Vector-memory loads complete in order:
        // the next tile was issued at the block's start, so it has landed
        // once only the filter loads of the last two units (2 * kFA each)
        // can still be outstanding.  No fence: this tile's pixel fragments
        // have all been read into registers, and the barrier alone makes
        // every wave's part of the next tile visible.
        __builtin_amdgcn_s_waitcnt(0x0F70 | (4 * kFA));
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
        const int t = cur_off;
        cur_off = nxt_off;
        nxt_off = t;
#pragma unroll
        for (int j = 0; j < PB; ++j) rb[j] = cur_off + lane_base[j];
        read_b(b_even, rb, 0);
      }
    }
  } else {
    const unsigned char* cur = bufs;
    unsigned char* nxt = bufs + buf_bytes;
    int chunk = 0, tap = 0, tap_r = 0, tap_c = 0, sub = 0;
    int tap_slots = 0;  // slot offset of the current tap: r * Wh + s
    // Pixel fragments of reduction step `ks` (0 .. KS-1) of a tap.
    auto load_b = [&](half8 (&b)[PB], int slots, int ks) {
      const int offset = slots * SLOTB + (2 * ks + khalf) * 16;
#pragma unroll
      for (int j = 0; j < PB; ++j)
        b[j] = *reinterpret_cast<const half8*>(cur + b_slot[j] * SLOTB + offset);
    };
    load_b(b_even, 0, 0);

    // One unit.  Pixel fragments of a reduction step are read from LDS while
    // the MFMAs of the step before run; the loads of the next channel block's
    // tile start in the first unit of a block.  The scheduling barriers keep
    // the compiler from sinking these prefetches below the MFMAs that hide
    // their latency.
    auto do_unit = [&](half8 (&a_use)[2][kFA], half8 (&a_fill)[2][kFA]) {
      const int slots = tap_slots;
      const int ks0 = 2 * sub;
      const bool tap_ends = sub + 1 == UPT;
      const bool last = tap_ends && tap + 1 == taps;
      int next_ks = ks0 + 2;
      if (tap_ends) {
        if (++tap_c == g.win_cols) { tap_c = 0; ++tap_r; }
        // After the last tap the tiles swap and the fragment is read again;
        // any slot inside the tile will do here.
        tap_slots = last ? 0 : tap_r * g.halo_cols + tap_c;
        next_ks = 0;
      }
      load_a(a_fill, step + 2 * (DEPTH - 1));
      if constexpr (MULTI) {
        if (tap == 0 && sub == 0 && chunk + 1 < n_chunks) {
          __builtin_amdgcn_sched_barrier(0);
          start_tile(nxt, static_cast<unsigned>((chunk + 1) * KC * 2));
        }
      }
      load_b(b_odd, slots, ks0 + 1);
      __builtin_amdgcn_sched_barrier(0);
      mfma_step(a_use[0], b_even);
      __builtin_amdgcn_sched_barrier(0);
      load_b(b_even, tap_slots, next_ks);
      __builtin_amdgcn_sched_barrier(0);
      mfma_step(a_use[1], b_odd);
      __builtin_amdgcn_sched_barrier(0);
      step += 2;
      if (last) {
        if constexpr (MULTI) {
          // End of the channel block.  Vector-memory loads complete in order:
          // the next tile was issued before the filter loads of all units but
          // the first, so it has landed once only the last two units' filter
          // loads (four each) can still be outstanding.  No fence: this
          // tile's pixel fragments have all been read into registers, and
          // the barrier alone makes every wave's part of the next tile
          // visible.
          if (units_per_chunk >= 3)
            __builtin_amdgcn_s_waitcnt(kWaitVm8);
          else if (units_per_chunk == 2)
            __builtin_amdgcn_s_waitcnt(kWaitVm4);
          else
            __builtin_amdgcn_s_waitcnt(kWaitVm0);
          __builtin_amdgcn_sched_barrier(0);
          __builtin_amdgcn_s_barrier();
          __builtin_amdgcn_sched_barrier(0);
          unsigned char* const t = const_cast<unsigned char*>(cur);
          cur = nxt;
          nxt = t;
          ++chunk;
          load_b(b_even, 0, 0);
        }
        tap = 0;
        tap_r = 0;
        tap_c = 0;
        sub = 0;
      } else if (tap_ends) {
        ++tap;
        sub = 0;
      } else {
        ++sub;
      }
    };

    int done = 0;
    for (; done + DEPTH <= total_units; done += DEPTH) {
#pragma unroll
      for (int d = 0; d < DEPTH; ++d)
        do_unit(a_buf[d], a_buf[(d + DEPTH - 1) % DEPTH]);
    }
#pragma unroll
    for (int d = 0; d + 1 < DEPTH; ++d)
      if (done + d < total_units)
        do_unit(a_buf[d], a_buf[(d + DEPTH - 1) % DEPTH]);

  }

  const __amdgpu_buffer_rsrc_t dst_rsrc = make_rsrc(dst, dst_bytes);
  const unsigned row_bytes = static_cast<unsigned>(g.features) * 2u;
#pragma unroll
  for (int j = 0; j < PB; ++j) {
    const unsigned pix_off =
        out_pixel[j] >= 0 ? static_cast<unsigned>(out_pixel[j]) * row_bytes
                          : kOob;
#pragma unroll
    for (int i = 0; i < kFA; ++i) {
      const unsigned off =
          pix_off + static_cast<unsigned>((fb0 + i) * 32 + 16 * khalf) * 2u;
      half8 lo, hi;
#pragma unroll
      for (int v = 0; v < 8; ++v) {
        lo[v] = static_cast<_Float16>(acc[i][j][v]);
        hi[v] = static_cast<_Float16>(acc[i][j][8 + v]);
      }
      __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(uint4v, lo),
                                             dst_rsrc, off, 0, kStoreAux);
      __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(uint4v, hi),
                                             dst_rsrc, off + 16u, 0, kStoreAux);
    }
  }
}

struct RowTilePlan {
  RowTile g;
  int wf = 0;            // feature groups of 64 per work-group
  int wp = 0;            // pixel groups of PB * 32 per work-group
  int pb = 0;            // pixel blocks of 32 per wave
  int kc = 0;            // channels per LDS tile
  size_t lds_bytes = 0;  // 0: shape not supported
  long score = 0;
  unsigned n_groups = 0;
};

// Geometry for work-groups of `tile_pixels` consecutive output pixels;
// lds_bytes == 0 when the tile does not fit.  The score estimates the useful
// pixels resident on a compute unit: work-groups that fit its LDS (at most two
// waves per SIMD) times the pixels of a tile, discounted by the unused part
// of the wave tiles.
RowTilePlan plan_tile(const snn_hip_conv2d_params& p, int wf, int wp, int pb,
                      int kc, int tile_pixels) {
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
  g.n_fslices = p.features / (64 * wf);
  const int n_chunks = p.channels / kc;
  const size_t slot_bytes = static_cast<size_t>(kc) * 2 + 16;
  const size_t n_blocks = ceil_div(g.n_slots * slot_bytes, size_t{1024});
  const size_t n_table = n_blocks * 1024 / slot_bytes + 1;
  const size_t lds_bytes =
      (n_chunks > 1 ? 2 : 1) * n_blocks * 1024 + n_table * 4;
  if (lds_bytes > kMaxLdsBytes) return plan;
  plan.wf = wf; plan.wp = wp; plan.pb = pb; plan.kc = kc;
  plan.lds_bytes = lds_bytes;
  const long resident =
      std::min<long>(kMaxLdsBytes / lds_bytes, 8 / (wf * wp));
  plan.score = resident * tile_pixels * tile_pixels / (wp * pb * 32);
  plan.n_groups = static_cast<unsigned>(n_tiles) *
                  static_cast<unsigned>(g.n_fslices);
  return plan;
}

// Tile sizes tried: the full capacity of the work-group (tiles then start
// anywhere in a row), and every whole number of rows below it.
RowTilePlan best_tile(const snn_hip_conv2d_params& p, int wf, int wp, int pb,
                      int kc) {
  const int total = p.batch * p.out_rows * p.out_cols;
  const int capacity = std::min(wp * pb * 32, total);
  RowTilePlan best = plan_tile(p, wf, wp, pb, kc, capacity);
  for (int rows = capacity / p.out_cols; rows >= 1; --rows) {
    const RowTilePlan plan = plan_tile(p, wf, wp, pb, kc, rows * p.out_cols);
    if (plan.lds_bytes != 0 && plan.score > best.score) best = plan;
  }
  return best;
}

// One channel block: 64 channels per LDS tile.  Otherwise 32, so that two
// double-buffered work-groups fit the LDS of a compute unit.  Waves own 64 features x 128
// pixels when that makes at least 1.5 waves per SIMD, else 64 x 64; the
// work-group is four waves when at least three work-groups per compute unit
// result, else two.
RowTilePlan compute_plan(const snn_hip_conv2d_params& p);

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

RowTilePlan compute_plan(const snn_hip_conv2d_params& p) {
  const int kc = p.channels == 64 ? 64 : 32;
  const int wf = p.features % 128 == 0 ? 2 : 1;
  const long pixels = static_cast<long>(p.batch) * p.out_rows * p.out_cols;
  const long wave_tiles = (pixels + 127) / 128 * (p.features / 64);
  const int pb = wave_tiles >= 1536 ? 4 : 2;
  const RowTilePlan big = best_tile(p, wf, 4 / wf, pb, kc);
  if (big.lds_bytes != 0 && big.n_groups >= 768) return big;
  const RowTilePlan small = best_tile(p, wf, 2 / wf, pb, kc);
  return small.lds_bytes != 0 ? small : big;
}

template <int WF, int WP, int PB, int KC, bool MULTI, bool WIN3>
void launch_plan(const _Float16* input, const _Float16* wpk, _Float16* output,
                 const snn_hip_conv2d_params& p, const RowTilePlan& plan,
                 size_t wgt_elems, hipStream_t stream) {
  auto kernel = conv_rowtile_f16_kernel<WF, WP, PB, KC, MULTI, WIN3>;
  static const hipError_t attr = hipFuncSetAttribute(
      reinterpret_cast<const void*>(kernel),
      hipFuncAttributeMaxDynamicSharedMemorySize, kMaxLdsBytes);
  (void)attr;
  const size_t x = static_cast<size_t>(p.batch) * p.in_rows * p.in_cols *
                   p.channels;
  const size_t y = static_cast<size_t>(p.batch) * p.out_rows * p.out_cols *
                   p.features;
  KernelTimer timer(stream);
  hipLaunchKernelGGL(kernel, dim3(plan.n_groups), dim3(64 * WF * WP),
                     plan.lds_bytes, stream, input, wpk, output, plan.g,
                     static_cast<unsigned>(x * 2),
                     static_cast<unsigned>(wgt_elems * 2),
                     static_cast<unsigned>(y * 2), plan.n_groups);
}

template <int WF, int WP, int PB>
bool launch_shape(const _Float16* input, const _Float16* wpk,
                  _Float16* output, const snn_hip_conv2d_params& p,
                  const RowTilePlan& plan, size_t wgt_elems,
                  hipStream_t stream) {
  if (plan.wf != WF || plan.wp != WP || plan.pb != PB) return false;
  const bool multi = p.channels > plan.kc;
  const bool win3 = p.window_rows == 3 && p.window_cols == 3;
#define SNN_ROWTILE_CASE(KC, MULTI, WIN3)                                     \
  if (plan.kc == KC && multi == MULTI && win3 == WIN3) {                      \
    launch_plan<WF, WP, PB, KC, MULTI, WIN3>(input, wpk, output, p, plan,     \
                                             wgt_elems, stream);              \
    return true;                                                              \
  }
  SNN_ROWTILE_CASE(64, false, true)
  SNN_ROWTILE_CASE(32, true, true)
  SNN_ROWTILE_CASE(64, false, false)
  SNN_ROWTILE_CASE(32, true, false)
#undef SNN_ROWTILE_CASE
  return false;
}

}  // namespace

bool conv2d_rowtile_f16_supports(const snn_hip_conv2d_params& p) {
  const size_t x = static_cast<size_t>(p.batch) * p.in_rows * p.in_cols *
                   p.channels;
  const size_t y = static_cast<size_t>(p.batch) * p.out_rows * p.out_cols *
                   p.features;
  if (p.stride_rows != 1 || p.stride_cols != 1) return false;
  if (p.channels % 64 != 0 || p.features % 64 != 0) return false;
  // 1x1 windows have no taps to reuse an LDS tile over: the implicit-GEMM
  // kernel measured as fast or faster there.
  if (p.window_rows * p.window_cols == 1) return false;
  if ((x > y ? x : y) * 2 > kMaxBufferBytes) return false;
  return make_plan(p).lds_bytes != 0;
}

int launch_conv2d_rowtile_f16(const _Float16* input, const _Float16* filter,
                              _Float16* output, const snn_hip_conv2d_params& p,
                              _Float16* packed, hipStream_t stream,
                              bool transposed_filter) {
  const RowTilePlan plan = make_plan(p);
  if (plan.lds_bytes == 0) return SNN_HIP_INVALID_ALGORITHM;
  static const bool print_plan = SNN_TUNING_ENV("SNN_HIP_F16_PLAN") != nullptr;
  if (print_plan)
    fprintf(stderr,
            "rowtile f16: waves %dx%d, %d pixel blocks, %d channels/tile, "
            "%d pixels/tile, %u work-groups, %zu B LDS\n",
            plan.wf, plan.wp, plan.pb, plan.kc, plan.g.tile_pixels,
            plan.n_groups, plan.lds_bytes);
  const int taps = p.window_rows * p.window_cols;
  const size_t wgt_elems =
      static_cast<size_t>(taps) * p.channels * p.features;
  hipLaunchKernelGGL(
      pack_filter_rowtile_kernel,
      dim3(static_cast<unsigned>(ceil_div(wgt_elems / 8, size_t{256}))),
      dim3(256), 0, stream, filter, packed, p.channels, p.features, taps,
      plan.kc, static_cast<int>(wgt_elems / 8), transposed_filter);
  const bool launched =
      launch_shape<1, 2, 2>(input, packed, output, p, plan, wgt_elems, stream) ||
      launch_shape<1, 2, 4>(input, packed, output, p, plan, wgt_elems, stream) ||
      launch_shape<1, 4, 2>(input, packed, output, p, plan, wgt_elems, stream) ||
      launch_shape<1, 4, 4>(input, packed, output, p, plan, wgt_elems, stream) ||
      launch_shape<2, 1, 2>(input, packed, output, p, plan, wgt_elems, stream) ||
      launch_shape<2, 1, 4>(input, packed, output, p, plan, wgt_elems, stream) ||
      launch_shape<2, 2, 2>(input, packed, output, p, plan, wgt_elems, stream) ||
      launch_shape<2, 2, 4>(input, packed, output, p, plan, wgt_elems, stream);
  if (!launched) return SNN_HIP_INVALID_ALGORITHM;
  const hipError_t err = hipGetLastError();
  if (err != hipSuccess) return report_hip_error(err, "conv_rowtile_f16_kernel");
  return SNN_HIP_OK;
}

}  // namespace snn
