// Half-precision filter gradient of 3x3 stride-1 SAME convolutions (and, at
// the end of the file, of 1x1 ones) on the binary16 matrix cores (gfx950).
//
//   dW[r][s][c][k] = sum over (n, oy, ox) of X[n][oy+r-1][ox+s-1][c] * dY[n][oy][ox][k]
//
// (the FilterBackprop direction of sycldnn::conv2d::launch,
// include/portdnn/conv2d/launch.h:59-118; products of binary16 values summed
// in fp32 and rounded to binary16 once).
//
// The reduction runs over pixels, which is the slow dimension of both
// operands in memory (NHWC), while v_mfma_f32_32x32x16_f16 wants eight
// consecutive reduction indices per lane.  ds_read_b64_tr_b16 does that
// transposition on the way out of LDS: within 16 lanes, lane 4 j + i supplies
// the address of four consecutive halves (columns 4 i ... 4 i + 3) of row j,
// and lane t receives column t of rows 0 ... 3.  Two such reads make one
// operand.
//
//   * A work-group (4 waves, one per SIMD, one work-group per CU) owns a
//     64-channel x 64-feature tile of dW for all nine taps -- wave w a 32 x 32
//     quarter of it, nine 32 x 32 accumulator blocks -- and walks a run of
//     consecutive bands of output rows.  (A single wave issues the 32 x 32 x 16
//     instruction at its full rate, the 16 x 16 x 32 one at 0.56 of it.)
//   * A band's input rows (with the halo and zero padding, row pitch
//     cols + 2 pixels) and dY rows (same pitch, zeros in the two extra
//     columns) are loaded into LDS with 16-byte LDS-direct loads, padding
//     through the buffer bounds.  With equal pitches the tap (r, s) operand of
//     pixel m is the input pixel m + r * pitch + s: one flat run of pixels per
//     band, cut into chunks of 16, whatever the image width.  Two LDS
//     buffers: the next band arrives while this one is multiplied.
//   * Per chunk and wave: one dY operand (2 transposing reads) + per filter
//     row 12 consecutive input pixels (3 reads), whose windows at pixel 0, 1
//     and 2 are the row's three taps (one funnel shift per register for the
//     middle one): 11 reads, fetched one chunk ahead, feed 9 matrix
//     instructions.  A wave issues one such read per 32 cycles (measured), a
//     32x32x16 instruction takes 32.
//   * 16-byte pieces of a pixel are XOR-swizzled on the way in so that the 16
//     lanes of a transposing read (4 pixels x 32 bytes) fall into distinct
//     banks.
//   * Float atomics retire one lane at a time (measured: 19 M of them cost
//     60 us), so the partial tiles are stored, and a second kernel sums them
//     and rounds to binary16.

#include "snn_common.h"
#include "snn_kernels.h"

namespace snn {

namespace {

typedef float float4v __attribute__((ext_vector_type(4)));
typedef float float16v __attribute__((ext_vector_type(16)));
typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef short short4v __attribute__((ext_vector_type(4)));
typedef short short8v __attribute__((ext_vector_type(8)));
typedef unsigned uint2v __attribute__((ext_vector_type(2)));
typedef unsigned uint4v __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) void* lds_ptr;
typedef __attribute__((address_space(3))) short4v* lds_short4_ptr;

constexpr int kWaves = 4;
constexpr int kTile = 64;         // channels and features per work-group
constexpr int kTaps = 9;
constexpr int kChunk = 16;        // pixels per matrix instruction
constexpr int kPixelBytes = 128;  // 64 halves
constexpr int kTileFloats = kTaps * kTile * kTile;
constexpr int kBufBytes = 78 * 1024;  // one of the two LDS buffers
constexpr int kNumCus = 256;
constexpr int kReduceGroups = 16;  // partial sums per output in the reduction
constexpr unsigned kOobOffset = 0x7FFFFFF0u;  // beyond every buffer's range
constexpr size_t kMaxBufferBytes = 0x7FFFFFF0u;

struct FbGeom {
  int batch, rows, cols, channels, features;
  int pitch;            // cols + 2
  unsigned pitch_magic; // ceil(2^32 / pitch)
  int band;             // output rows per band
  int bands_per_image;
  int n_subbands;       // batch * bands_per_image
  int group;            // bands per task (several whole images when small)
  int n_tasks;
  int x_px;             // LDS pixels of a band's input rows (multiple of 32)
  int y_px;             // LDS pixels of a band's dY rows (multiple of 32)
  int c_tiles, k_tiles, n_splits;
  int per_split;        // consecutive tasks per work-group
};

__device__ inline __amdgpu_buffer_rsrc_t make_rsrc(const void* p,
                                                   size_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0,
                                           static_cast<unsigned>(bytes),
                                           0x00020000);
}

constexpr int vmcnt_imm(int n) {
  return 0x0F70 | (n & 15) | ((n >> 4) << 14);
}

// Which 16-byte position of LDS pixel p holds 16-byte piece c: c ^ swz(p).
// Four consecutive pixels get four different piece pairs, and pixels 8 apart
// swap the pairs of even and odd pixels.
__device__ __forceinline__ unsigned swz(unsigned p) {
  return ((p & 3u) ^ ((p >> 3) & 1u)) << 1;
}

__device__ __forceinline__ half8 read_transposed(const char* at_lo,
                                                 const char* at_hi) {
  const short4v lo =
      __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4_ptr)(at_lo));
  const short4v hi =
      __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4_ptr)(at_hi));
  const short8v both =
      __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  return __builtin_bit_cast(half8, both);
}

__device__ __forceinline__ uint2v read_transposed4(const char* at) {
  return __builtin_bit_cast(
      uint2v, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4_ptr)(at)));
}

// part: [split][tile] tiles of 9 x 64 x 64 floats in accumulator order, each
// written once.
__global__ void __launch_bounds__(64 * kWaves)
    conv_filter_backprop_3x3_f16_kernel(const _Float16* __restrict__ x,
                                        const _Float16* __restrict__ dy,
                                        float* __restrict__ part, FbGeom g) {
  // two objects, so that the compiler ties an LDS read to the loads of its
  // own buffer only
  __shared__ __align__(1024) char buf0[kBufBytes];
  __shared__ __align__(1024) char buf1[kBufBytes];
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int n_tiles = g.c_tiles * g.k_tiles;
  const int tile = blockIdx.x % n_tiles;
  const int split = blockIdx.x / n_tiles;
  const int ct = tile % g.c_tiles;
  const int kt = tile / g.c_tiles;

  const __amdgpu_buffer_rsrc_t x_rsrc = make_rsrc(
      x, static_cast<size_t>(g.batch) * g.rows * g.cols * g.channels * 2);
  const __amdgpu_buffer_rsrc_t dy_rsrc = make_rsrc(
      dy, static_cast<size_t>(g.batch) * g.rows * g.cols * g.features * 2);

  const int sb_px = g.x_px + g.y_px;  // LDS pixels per band

  // ---- transposing-read offsets, relative to the chunk's first pixel ------
  // v_mfma_f32_32x32x16_f16: lane l holds row (or column) l % 32 at reduction
  // indices 8 (l / 32) ... + 7.  Of lane = 16 gq + 4 j + e, as a source of the
  // transposing read: pixel 8 (gq / 2) + j (+ 4 for the second read), halves
  // 4 e ... 4 e + 3 of the 16-wide block gq % 2 of this wave's 32.
  const unsigned gq = lane >> 4, j = (lane >> 2) & 3, e = lane & 3;
  const unsigned c32 = wave & 1, k32 = wave >> 1;
  // Input operands: per filter row three reads of 4 pixels (12 consecutive
  // pixels per lane); the three taps of the row are the 8-pixel windows at
  // pixel 0, 1 and 2 of them.  (A wave can issue one such read per 32 cycles:
  // 11 reads per chunk instead of 20 keep it near the matrix rate.)
  unsigned off_x[3][3];
  unsigned off_y[2];
#pragma unroll
  for (int h = 0; h < 3; ++h) {
    const unsigned p0 = 8 * (gq >> 1) + 4 * h + j;
#pragma unroll
    for (int r = 0; r < 3; ++r) {
      const unsigned p = r * g.pitch + p0;
      off_x[r][h] =
          p * kPixelBytes +
          (((4 * c32 + 2 * (gq & 1) + (e >> 1)) ^ swz(p)) << 4) + ((e & 1) << 3);
    }
    if (h < 2)
      off_y[h] = (g.x_px + p0) * kPixelBytes +
                 (((4 * k32 + 2 * (gq & 1) + (e >> 1)) ^ swz(p0)) << 4) +
                 ((e & 1) << 3);
  }

  // acc[tap][i]: feature 32 k32 + 8 (i / 4) + 4 (lane / 32) + i % 4,
  // channel 32 c32 + lane % 32
  float16v acc[kTaps];
#pragma unroll
  for (int tap = 0; tap < kTaps; ++tap)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[tap][i] = 0.f;

  const unsigned lane_px = lane >> 3;   // pixel of a load instruction's eight
  const unsigned lane_piece = lane & 7; // 16-byte position within the pixel
  const int n_chunks = g.y_px / kChunk;

  // Every band has the same shape, so what a load instruction of this wave
  // fetches is fixed relative to the band's first output row: its row (for
  // the test against the image's top and bottom) and its byte offset are
  // worked out once (a load then costs a handful of vector instructions
  // instead of thirty, which nothing hides with one wave per SIMD).
  constexpr int kMaxXLoads = 20, kMaxYLoads = 10;  // per wave: 78 KB buffers
  const int x_loads = g.x_px / 8, y_loads = g.y_px / 8;
  int x_row[kMaxXLoads], x_rel[kMaxXLoads], y_row[kMaxYLoads], y_rel[kMaxYLoads];
#pragma unroll
  for (int idx = 0; idx < kMaxXLoads; ++idx) {
    const unsigned p = 8 * (wave + kWaves * idx) + lane_px;
    const unsigned row = __umulhi(p, g.pitch_magic);
    const int ix = static_cast<int>(p - row * g.pitch) - 1;
    const bool ok = row < static_cast<unsigned>(g.band + 2) && ix >= 0 &&
                    ix < g.cols;
    // rows outside [-1, band] fail every test against the image
    x_row[idx] = ok ? static_cast<int>(row) - 1 : -0x40000000;
    x_rel[idx] = (((static_cast<int>(row) - 1) * g.cols + ix) * g.channels +
                  ct * kTile) * 2 +
                 static_cast<int>((lane_piece ^ swz(p)) << 4);
  }
#pragma unroll
  for (int idx = 0; idx < kMaxYLoads; ++idx) {
    const unsigned p = 8 * (wave + kWaves * idx) + lane_px;
    const unsigned row = __umulhi(p, g.pitch_magic);
    const int col = static_cast<int>(p - row * g.pitch);
    const bool ok = row < static_cast<unsigned>(g.band) && col < g.cols;
    y_row[idx] = ok ? static_cast<int>(row) : -0x40000000;
    y_rel[idx] = ((static_cast<int>(row) * g.cols + col) * g.features +
                  kt * kTile) * 2 +
                 static_cast<int>((lane_piece ^ swz(p)) << 4);
  }

  auto issue_task = [&](int task, char* buf) {
    for (int i = 0; i < g.group; ++i) {
      const int sb = task * g.group + i;
      const bool live = sb < g.n_subbands;
      const int n = sb / g.bands_per_image;
      const int oy0 = (sb - n * g.bands_per_image) * g.band;
      // rows of the image, relative to oy0; none when the band is past the end
      const int lo = live ? -oy0 : 1, hi = live ? g.rows - oy0 : 0;
      const int x_base = (n * g.rows + oy0) * g.cols * g.channels * 2;
      const int y_base = (n * g.rows + oy0) * g.cols * g.features * 2;
      char* base = buf + i * sb_px * kPixelBytes;
#pragma unroll
      for (int idx = 0; idx < kMaxXLoads; ++idx) {
        const int l = wave + kWaves * idx;
        if (l < x_loads) {
          const bool ok = x_row[idx] >= lo && x_row[idx] < hi;
          __builtin_amdgcn_raw_ptr_buffer_load_lds(
              x_rsrc, (lds_ptr)(base + l * 1024), 16,
              ok ? static_cast<unsigned>(x_base + x_rel[idx]) : kOobOffset, 0,
              0, 0);
        }
      }
      char* ybase = base + g.x_px * kPixelBytes;
#pragma unroll
      for (int idx = 0; idx < kMaxYLoads; ++idx) {
        const int l = wave + kWaves * idx;
        if (l < y_loads) {
          const bool ok = y_row[idx] >= lo && y_row[idx] < hi;
          __builtin_amdgcn_raw_ptr_buffer_load_lds(
              dy_rsrc, (lds_ptr)(ybase + l * 1024), 16,
              ok ? static_cast<unsigned>(y_base + y_rel[idx]) : kOobOffset, 0,
              0, 0);
        }
      }
    }
  };

  auto fetch = [&](const char* at, half8& ya, uint2v (&xw)[3][3]) {
    ya = read_transposed(at + off_y[0], at + off_y[1]);
#pragma unroll
    for (int r = 0; r < 3; ++r)
#pragma unroll
      for (int h = 0; h < 3; ++h) xw[r][h] = read_transposed4(at + off_x[r][h]);
  };
  // The windows are cut out of the 12 pixels here, a chunk after the reads
  // were issued, so that nothing waits on them.
  auto multiply = [&](const half8& ya, const uint2v (&xw)[3][3]) {
#pragma unroll
    for (int r = 0; r < 3; ++r) {
      const unsigned w0 = xw[r][0][0], w1 = xw[r][0][1], w2 = xw[r][1][0],
                     w3 = xw[r][1][1], w4 = xw[r][2][0];
      const uint4v s0 = {w0, w1, w2, w3};
      const uint4v s1 = {__builtin_amdgcn_alignbit(w1, w0, 16),
                         __builtin_amdgcn_alignbit(w2, w1, 16),
                         __builtin_amdgcn_alignbit(w3, w2, 16),
                         __builtin_amdgcn_alignbit(w4, w3, 16)};
      const uint4v s2 = {w1, w2, w3, w4};
      acc[3 * r] = __builtin_amdgcn_mfma_f32_32x32x16_f16(
          ya, __builtin_bit_cast(half8, s0), acc[3 * r], 0, 0, 0);
      acc[3 * r + 1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(
          ya, __builtin_bit_cast(half8, s1), acc[3 * r + 1], 0, 0, 0);
      acc[3 * r + 2] = __builtin_amdgcn_mfma_f32_32x32x16_f16(
          ya, __builtin_bit_cast(half8, s2), acc[3 * r + 2], 0, 0, 0);
    }
  };

  // Chunks of the task's live bands, operands fetched one chunk ahead (the
  // last fetch repeats the last chunk).
  auto multiply_task = [&](int task, const char* buf) {
    const int live = min(g.group, g.n_subbands - task * g.group);
    const int total = live * n_chunks;
    half8 ya0, ya1;
    uint2v xb0[3][3], xb1[3][3];
    int next_px = 0, next_chunk = 0, fetched = 0;
    auto advance = [&]() {
      if (fetched + 1 < total) {
        ++fetched;
        next_px += kChunk;
        if (++next_chunk == n_chunks) {
          next_chunk = 0;
          next_px += g.x_px;
        }
      }
    };
    // (fences: the compiler otherwise sinks the reads next to their uses and
    // waits out the LDS latency twice per chunk)
    fetch(buf, ya0, xb0);
    for (int f = 0; f < total; f += 2) {
      advance();
      __builtin_amdgcn_sched_barrier(0);
      fetch(buf + next_px * kPixelBytes, ya1, xb1);
      __builtin_amdgcn_sched_barrier(0);
      multiply(ya0, xb0);
      if (f + 1 >= total) break;
      advance();
      __builtin_amdgcn_sched_barrier(0);
      fetch(buf + next_px * kPixelBytes, ya0, xb0);
      __builtin_amdgcn_sched_barrier(0);
      multiply(ya1, xb1);
    }
  };

  // ---- bands: load one ahead ------------------------------------------------
#define SNN_FILBK_STEP(cur, nxt)                              \
  {                                                           \
    if (task >= task_end) break;                              \
    __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));                 \
    __syncthreads();                                          \
    if (task + 1 < task_end) issue_task(task + 1, nxt);       \
    multiply_task(task, cur);                                 \
    ++task;                                                   \
  }
  // consecutive bands: the halo rows a band shares with the one before it
  // are still in this XCD's L2
  int task = split * g.per_split;
  const int task_end = min(g.n_tasks, task + g.per_split);
  if (task < task_end) issue_task(task, buf0);
  for (;;) {
    SNN_FILBK_STEP(buf0, buf1)
    SNN_FILBK_STEP(buf1, buf0)
  }
#undef SNN_FILBK_STEP

  // ---- store the partial tile ------------------------------------------------
  float* out = part + (static_cast<size_t>(split) * n_tiles + tile) * kTileFloats;
  // in accumulator order, [tap][wave][i4][lane] float4: every store
  // instruction writes 1 KB of consecutive memory
#pragma unroll
  for (int tap = 0; tap < kTaps; ++tap)
#pragma unroll
    for (int i4 = 0; i4 < 4; ++i4) {
      const float4v v = {acc[tap][4 * i4], acc[tap][4 * i4 + 1],
                         acc[tap][4 * i4 + 2], acc[tap][4 * i4 + 3]};
      *reinterpret_cast<float4v*>(
          out + (((tap * kWaves + wave) * 4 + i4) * 64 + lane) * 4) = v;
    }
}

// Sums the partial tiles and rounds: a work-group is 256 / n_groups
// consecutive float4 of the filter x n_groups groups of splits (a power of two
// up to 16).
__global__ void __launch_bounds__(256)
    filter_backprop_f16_reduce_kernel(const float4v* __restrict__ part,
                                      _Float16* __restrict__ dw, int n_tiles,
                                      int c_tiles, int n_splits, int n_groups,
                                      int channels, int features) {
  __shared__ float4v sums[256];
  constexpr int kTileVecs = kTileFloats / 4;
  const int width = 256 / n_groups;
  const int lane_o = threadIdx.x % width;
  const int group = threadIdx.x / width;
  const unsigned o = blockIdx.x * width + lane_o;  // float4 of the whole filter
  const unsigned tile = o / kTileVecs;
  const unsigned local = o - tile * kTileVecs;
  float4v sum = {0.f, 0.f, 0.f, 0.f};
  for (int sp = group; sp < n_splits; sp += n_groups)
    sum += part[(static_cast<size_t>(sp) * n_tiles + tile) * kTileVecs + local];
  sums[threadIdx.x] = sum;
  __syncthreads();
  if (group != 0) return;
  for (int i = 1; i < n_groups; ++i) sum += sums[i * width + lane_o];
  // accumulator order of the partial tiles: local = ((tap * 4 + wave) * 4 +
  // i4) * 64 + lane holds channel 32 (wave & 1) + lane % 32 and features
  // 32 (wave >> 1) + 8 i4 + 4 (lane / 32) ... + 3
  const unsigned ln = local & 63, i4 = (local >> 6) & 3, wv = (local >> 8) & 3;
  const unsigned tap = local >> 10;
  const unsigned c = 32 * (wv & 1) + (ln & 31);
  const unsigned k4 = 8 * (wv >> 1) + 2 * i4 + (ln >> 5);
  const unsigned ct = tile % c_tiles, kt = tile / c_tiles;
  typedef _Float16 half4v __attribute__((ext_vector_type(4)));
  half4v r;
#pragma unroll
  for (int v = 0; v < 4; ++v) r[v] = static_cast<_Float16>(sum[v]);
  *reinterpret_cast<half4v*>(
      dw + (static_cast<size_t>(tap) * channels + ct * kTile + c) * features +
      kt * kTile + 4 * k4) = r;
}

int round_up(int a, int b) { return ceil_div(a, b) * b; }

bool make_geom(const snn_hip_conv2d_params& p, FbGeom* g) {
  if (p.window_rows != 3 || p.window_cols != 3 || p.stride_rows != 1 ||
      p.stride_cols != 1 || p.pad_rows != 1 || p.pad_cols != 1 ||
      p.out_rows != p.in_rows || p.out_cols != p.in_cols)
    return false;
  if (p.channels % kTile != 0 || p.features % kTile != 0 || p.batch < 1)
    return false;
  const size_t x_bytes = static_cast<size_t>(p.batch) * p.in_rows * p.in_cols *
                         p.channels * 2;
  const size_t y_bytes = static_cast<size_t>(p.batch) * p.in_rows * p.in_cols *
                         p.features * 2;
  if (x_bytes > kMaxBufferBytes || y_bytes > kMaxBufferBytes) return false;
  g->batch = p.batch; g->rows = p.in_rows; g->cols = p.in_cols;
  g->channels = p.channels; g->features = p.features;
  g->pitch = p.in_cols + 2;
  g->pitch_magic = 0xFFFFFFFFu / static_cast<unsigned>(g->pitch) + 1u;
  // the most rows whose band fits a buffer, then evened out over the image
  auto band_px = [&](int band, int* x_px, int* y_px) {
    *y_px = round_up(band * g->pitch, kChunk);
    // (the third read of a row reaches two pixels past the last window)
    *x_px = round_up(*y_px + 2 * g->pitch + 4, kChunk);
    return *x_px + *y_px;
  };
  int x_px = 0, y_px = 0, band = 0;
  for (int r = 1; r <= p.in_rows; ++r) {
    if (band_px(r, &x_px, &y_px) * kPixelBytes > kBufBytes) break;
    band = r;
  }
  if (band == 0) return false;
  g->bands_per_image = ceil_div(p.in_rows, band);
  g->band = ceil_div(p.in_rows, g->bands_per_image);
  const int sb_px = band_px(g->band, &x_px, &y_px);
  g->x_px = x_px; g->y_px = y_px;
  g->n_subbands = p.batch * g->bands_per_image;
  g->group = 1;
  if (g->bands_per_image == 1)
    g->group = max(1, min(p.batch, kBufBytes / (sb_px * kPixelBytes)));
  g->n_tasks = ceil_div(g->n_subbands, g->group);
  g->c_tiles = p.channels / kTile;
  g->k_tiles = p.features / kTile;
  const int n_tiles = g->c_tiles * g->k_tiles;
  const int want = max(1, min(g->n_tasks, kNumCus / n_tiles));
  g->per_split = ceil_div(g->n_tasks, want);
  g->n_splits = ceil_div(g->n_tasks, g->per_split);
  return true;
}

// ---------------------------------------------------------------------------
// 1x1 (stride 1, no padding): dW[c][k] = sum over pixels m of X[m][c] * dY[m][k],
// one flat stream of pixels.  A work-group (4 waves, 2 x 2) owns a tile of
// (64 A) channels x (64 B) features of dW and a range of the pixels; wave
// (wc, wk) its quarter at (wc, wk), A x B blocks of 32 x 32.  Stages of 64
// pixels, [pixel][64 A channels] and [pixel][64 B features], arrive in two
// LDS buffers by LDS-direct loads (swizzled as
// above); per chunk of 16 pixels a wave fetches A + B operands for A x B
// matrix instructions.  The layers are bound by the bytes moved (the tile has
// 32 A B / (A + B) flop per loaded byte, and each work-group stores one
// partial tile), so the tile shape is picked to make loads plus partial
// tiles least.
struct Fb1Geom {
  int pixels, channels, features;
  int c_tiles, k_tiles, n_splits;
  int n_stages, per_split;  // stages of kStagePx pixels; consecutive per split
};
constexpr int kStagePx = 64;

template <int A, int B>
__device__ __forceinline__ void filter_backprop_1x1_body(
    const _Float16* __restrict__ x, const _Float16* __restrict__ dy,
    float* __restrict__ part, const Fb1Geom& g, char* buf0, char* buf1) {
  constexpr int kXBytes = 128 * A;  // per pixel
  constexpr int kYBytes = 128 * B;
  constexpr int kXStage = kStagePx * kXBytes;
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int wc = wave & 1, wk = wave >> 1;
  const int n_tiles = g.c_tiles * g.k_tiles;
  const int tile = blockIdx.x % n_tiles;
  const int split = blockIdx.x / n_tiles;
  const int ct = tile % g.c_tiles;
  const int kt = tile / g.c_tiles;
  const __amdgpu_buffer_rsrc_t x_rsrc =
      make_rsrc(x, static_cast<size_t>(g.pixels) * g.channels * 2);
  const __amdgpu_buffer_rsrc_t dy_rsrc =
      make_rsrc(dy, static_cast<size_t>(g.pixels) * g.features * 2);

  // transposing-read offsets within a chunk (see the 3x3 kernel)
  const unsigned gq = lane >> 4, j = (lane >> 2) & 3, e = lane & 3;
  unsigned off_x[A][2], off_y[B][2];
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const unsigned p = 8 * (gq >> 1) + 4 * h + j;
#pragma unroll
    for (int i = 0; i < A; ++i) {
      const unsigned piece = 4 * (wc * A + i) + 2 * (gq & 1) + (e >> 1);
      off_x[i][h] = p * kXBytes + ((piece ^ swz(p)) << 4) + ((e & 1) << 3);
    }
#pragma unroll
    for (int i = 0; i < B; ++i) {
      const unsigned piece = 4 * (wk * B + i) + 2 * (gq & 1) + (e >> 1);
      off_y[i][h] =
          kXStage + p * kYBytes + ((piece ^ swz(p)) << 4) + ((e & 1) << 3);
    }
  }

  float16v acc[A][B];
#pragma unroll
  for (int ia = 0; ia < A; ++ia)
#pragma unroll
    for (int ib = 0; ib < B; ++ib)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[ia][ib][i] = 0.f;

  // a 1 KB load covers 8 / A pixels of X (8 / B of dY)
  auto issue_stage = [&](int stage, char* buf) {
    const unsigned m0 = static_cast<unsigned>(stage) * kStagePx;
    constexpr int kXPieces = 8 * A, kYPieces = 8 * B;
    for (int l = wave; l < kStagePx * kXPieces / 64; l += kWaves) {
      const unsigned p = (64 * l + lane) / kXPieces;
      const unsigned piece = (64 * l + lane) % kXPieces;
      const unsigned m = m0 + p;
      const unsigned off =
          (m * g.channels + ct * 64 * A) * 2u + ((piece ^ swz(p)) << 4);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(
          x_rsrc, (lds_ptr)(buf + l * 1024), 16,
          m < static_cast<unsigned>(g.pixels) ? off : kOobOffset, 0, 0, 0);
    }
    for (int l = wave; l < kStagePx * kYPieces / 64; l += kWaves) {
      const unsigned p = (64 * l + lane) / kYPieces;
      const unsigned piece = (64 * l + lane) % kYPieces;
      const unsigned m = m0 + p;
      const unsigned off =
          (m * g.features + kt * 64 * B) * 2u + ((piece ^ swz(p)) << 4);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(
          dy_rsrc, (lds_ptr)(buf + kXStage + l * 1024), 16,
          m < static_cast<unsigned>(g.pixels) ? off : kOobOffset, 0, 0, 0);
    }
  };

  auto multiply_stage = [&](const char* buf) {
    half8 xa[2][A], yb[2][B];
    auto fetch = [&](int chunk, half8 (&xo)[A], half8 (&yo)[B]) {
      const char* xat = buf + chunk * kChunk * kXBytes;
      const char* yat = buf + chunk * kChunk * kYBytes;
#pragma unroll
      for (int i = 0; i < A; ++i)
        xo[i] = read_transposed(xat + off_x[i][0], xat + off_x[i][1]);
#pragma unroll
      for (int i = 0; i < B; ++i)
        yo[i] = read_transposed(yat + off_y[i][0], yat + off_y[i][1]);
    };
    fetch(0, xa[0], yb[0]);
#pragma unroll
    for (int chunk = 0; chunk < kStagePx / kChunk; ++chunk) {
      __builtin_amdgcn_sched_barrier(0);
      if (chunk + 1 < kStagePx / kChunk)
        fetch(chunk + 1, xa[(chunk + 1) & 1], yb[(chunk + 1) & 1]);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int ia = 0; ia < A; ++ia)
#pragma unroll
        for (int ib = 0; ib < B; ++ib)
          acc[ia][ib] = __builtin_amdgcn_mfma_f32_32x32x16_f16(
              yb[chunk & 1][ib], xa[chunk & 1][ia], acc[ia][ib], 0, 0, 0);
    }
  };

#define SNN_FILBK1_STEP(cur, nxt)                               \
  {                                                             \
    if (stage >= stage_end) break;                              \
    __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));                   \
    __syncthreads();                                            \
    if (stage + 1 < stage_end) issue_stage(stage + 1, nxt);     \
    multiply_stage(cur);                                        \
    ++stage;                                                    \
  }
  int stage = split * g.per_split;
  const int stage_end = min(g.n_stages, stage + g.per_split);
  if (stage < stage_end) issue_stage(stage, buf0);
  for (;;) {
    SNN_FILBK1_STEP(buf0, buf1)
    SNN_FILBK1_STEP(buf1, buf0)
  }
#undef SNN_FILBK1_STEP

  // partial tile in accumulator order: [wave][ia][ib][i4][lane] float4
  float* out = part + (static_cast<size_t>(split) * n_tiles + tile) *
                          (4096 * A * B);
#pragma unroll
  for (int ia = 0; ia < A; ++ia)
#pragma unroll
    for (int ib = 0; ib < B; ++ib)
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4) {
        const float4v v = {acc[ia][ib][4 * i4], acc[ia][ib][4 * i4 + 1],
                           acc[ia][ib][4 * i4 + 2], acc[ia][ib][4 * i4 + 3]};
        *reinterpret_cast<float4v*>(
            out + ((((wave * A + ia) * B + ib) * 4 + i4) * 64 + lane) * 4) = v;
      }
}

// (plain functions around the template body: the compiler drops the host side
// of a kernel template whose body names the LDS-direct load)
#define SNN_FILBK1_KERNEL(A, B)                                              \
  __global__ void __launch_bounds__(64 * kWaves)                             \
      filter_backprop_1x1_f16_a##A##_b##B(const _Float16* __restrict__ x,    \
                                          const _Float16* __restrict__ dy,   \
                                          float* __restrict__ part,          \
                                          Fb1Geom g) {                       \
    __shared__ __align__(1024) char buf0[kStagePx * 128 * (A + B)];          \
    __shared__ __align__(1024) char buf1[kStagePx * 128 * (A + B)];          \
    filter_backprop_1x1_body<A, B>(x, dy, part, g, buf0, buf1);              \
  }
SNN_FILBK1_KERNEL(1, 1)
SNN_FILBK1_KERNEL(1, 2)
SNN_FILBK1_KERNEL(1, 4)
SNN_FILBK1_KERNEL(2, 2)
SNN_FILBK1_KERNEL(2, 4)
#undef SNN_FILBK1_KERNEL

// Sums the partial tiles of the 1x1 kernel and rounds.  Thread o of the
// filter's float4s, in accumulator order within a tile.
__global__ void __launch_bounds__(256)
    filter_backprop_1x1_f16_reduce_kernel(const float4v* __restrict__ part,
                                          _Float16* __restrict__ dw,
                                          int n_tiles, int c_tiles,
                                          int n_splits, int n_groups, int a,
                                          int b, int features) {
  __shared__ float4v sums[256];
  const int tile_vecs = 1024 * a * b;
  const int width = 256 / n_groups;
  const int lane_o = threadIdx.x % width;
  const int group = threadIdx.x / width;
  const unsigned o = blockIdx.x * width + lane_o;
  const unsigned tile = o / tile_vecs;
  const unsigned local = o - tile * tile_vecs;
  float4v sum = {0.f, 0.f, 0.f, 0.f};
  for (int sp = group; sp < n_splits; sp += n_groups)
    sum += part[(static_cast<size_t>(sp) * n_tiles + tile) * tile_vecs + local];
  sums[threadIdx.x] = sum;
  __syncthreads();
  if (group != 0) return;
  for (int i = 1; i < n_groups; ++i) sum += sums[i * width + lane_o];
  const unsigned ln = local & 63, i4 = (local >> 6) & 3;
  unsigned idx = local >> 8;
  const unsigned ib = idx % b; idx /= b;
  const unsigned ia = idx % a; idx /= a;
  const unsigned wc = idx & 1, wk = idx >> 1;
  const unsigned ct = tile % c_tiles, kt = tile / c_tiles;
  const unsigned c = ct * 64 * a + (wc * a + ia) * 32 + (ln & 31);
  const unsigned k = kt * 64 * b + (wk * b + ib) * 32 + 8 * i4 + 4 * (ln >> 5);
  typedef _Float16 half4v __attribute__((ext_vector_type(4)));
  half4v r;
#pragma unroll
  for (int v = 0; v < 4; ++v) r[v] = static_cast<_Float16>(sum[v]);
  *reinterpret_cast<half4v*>(dw + static_cast<size_t>(c) * features + k) = r;
}

struct Fb1Plan {
  int a = 0, b = 0;
  Fb1Geom g;
};

// The tile shape whose loads plus partial tiles (written and read back) come
// to the fewest bytes.
bool make_plan_1x1(const snn_hip_conv2d_params& p, Fb1Plan* plan) {
  if (p.window_rows != 1 || p.window_cols != 1 || p.stride_rows != 1 ||
      p.stride_cols != 1 || p.pad_rows != 0 || p.pad_cols != 0 ||
      p.out_rows != p.in_rows || p.out_cols != p.in_cols)
    return false;
  if (p.channels % 64 != 0 || p.features % 64 != 0 || p.batch < 1) return false;
  const size_t pixels = static_cast<size_t>(p.batch) * p.in_rows * p.in_cols;
  if (pixels * p.channels * 2 > kMaxBufferBytes ||
      pixels * p.features * 2 > kMaxBufferBytes)
    return false;
  static const int shapes[5][2] = {{1, 1}, {1, 2}, {1, 4}, {2, 2}, {2, 4}};
  double best = -1;
  for (const auto& sh : shapes) {
    const int a = sh[0], b = sh[1];
    if (p.channels % (64 * a) != 0 || p.features % (64 * b) != 0) continue;
    Fb1Geom g;
    g.pixels = static_cast<int>(pixels);
    g.channels = p.channels; g.features = p.features;
    g.c_tiles = p.channels / (64 * a);
    g.k_tiles = p.features / (64 * b);
    g.n_stages = ceil_div(g.pixels, kStagePx);
    const int n_tiles = g.c_tiles * g.k_tiles;
    const int want = max(1, min(g.n_stages, kNumCus / n_tiles));
    g.per_split = ceil_div(g.n_stages, want);
    g.n_splits = ceil_div(g.n_stages, g.per_split);
    const double loads = 2.0 * pixels *
                         (static_cast<double>(p.channels) * g.k_tiles +
                          static_cast<double>(p.features) * g.c_tiles);
    const double partials =
        2.0 * 4.0 * 4096.0 * a * b * n_tiles * g.n_splits;
    const double cost = loads + partials;
    if (best < 0 || cost < best) {
      best = cost;
      plan->a = a; plan->b = b; plan->g = g;
    }
  }
  return best >= 0;
}

}  // namespace

bool conv2d_filter_backprop_3x3_f16_supports(const snn_hip_conv2d_params& p) {
  FbGeom g;
  return make_geom(p, &g);
}

size_t conv2d_filter_backprop_3x3_f16_partial_floats(
    const snn_hip_conv2d_params& p) {
  FbGeom g;
  if (!make_geom(p, &g)) return 0;
  return static_cast<size_t>(g.n_splits) * g.c_tiles * g.k_tiles * kTileFloats;
}

// x, dy, dw 16-byte aligned; part holds
// conv2d_filter_backprop_3x3_f16_partial_floats(p) floats.
int launch_conv2d_filter_backprop_3x3_f16(const _Float16* x,
                                          const _Float16* dy, _Float16* dw,
                                          float* part,
                                          const snn_hip_conv2d_params& p,
                                          hipStream_t stream) {
  FbGeom g;
  if (!make_geom(p, &g)) return SNN_HIP_INVALID_ALGORITHM;
  const int n_tiles = g.c_tiles * g.k_tiles;
  {
    KernelTimer timer(stream);
    hipLaunchKernelGGL(conv_filter_backprop_3x3_f16_kernel,
                       dim3(static_cast<unsigned>(n_tiles * g.n_splits)),
                       dim3(64 * kWaves), 0, stream, x, dy, part, g);
  }
  const unsigned vecs = static_cast<unsigned>(n_tiles) * (kTileFloats / 4);
  int n_groups = 1;
  while (n_groups < kReduceGroups && 2 * n_groups <= g.n_splits) n_groups *= 2;
  hipLaunchKernelGGL(filter_backprop_f16_reduce_kernel,
                     dim3(vecs / (256 / n_groups)), dim3(256), 0, stream,
                     reinterpret_cast<const float4v*>(part), dw, n_tiles,
                     g.c_tiles, g.n_splits, n_groups, p.channels, p.features);
  return SNN_HIP_OK;
}

bool conv2d_filter_backprop_1x1_f16_supports(const snn_hip_conv2d_params& p) {
  Fb1Plan plan;
  return make_plan_1x1(p, &plan);
}

size_t conv2d_filter_backprop_1x1_f16_partial_floats(
    const snn_hip_conv2d_params& p) {
  Fb1Plan plan;
  if (!make_plan_1x1(p, &plan)) return 0;
  return static_cast<size_t>(plan.g.n_splits) * plan.g.c_tiles *
         plan.g.k_tiles * 4096 * plan.a * plan.b;
}

int launch_conv2d_filter_backprop_1x1_f16(const _Float16* x,
                                          const _Float16* dy, _Float16* dw,
                                          float* part,
                                          const snn_hip_conv2d_params& p,
                                          hipStream_t stream) {
  Fb1Plan plan;
  if (!make_plan_1x1(p, &plan)) return SNN_HIP_INVALID_ALGORITHM;
  const Fb1Geom& g = plan.g;
  const int n_tiles = g.c_tiles * g.k_tiles;
  void (*kernel)(const _Float16*, const _Float16*, float*, Fb1Geom) = nullptr;
  if (plan.a == 1 && plan.b == 1) kernel = filter_backprop_1x1_f16_a1_b1;
  if (plan.a == 1 && plan.b == 2) kernel = filter_backprop_1x1_f16_a1_b2;
  if (plan.a == 1 && plan.b == 4) kernel = filter_backprop_1x1_f16_a1_b4;
  if (plan.a == 2 && plan.b == 2) kernel = filter_backprop_1x1_f16_a2_b2;
  if (plan.a == 2 && plan.b == 4) kernel = filter_backprop_1x1_f16_a2_b4;
  if (kernel == nullptr) return SNN_HIP_INVALID_ALGORITHM;
  {
    KernelTimer timer(stream);
    hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned>(n_tiles * g.n_splits)),
                       dim3(64 * kWaves), 0, stream, x, dy, part, g);
  }
  const int tile_vecs = 1024 * plan.a * plan.b;
  const unsigned vecs = static_cast<unsigned>(n_tiles) * tile_vecs;
  int n_groups = 1;
  while (n_groups < kReduceGroups && 2 * n_groups <= g.n_splits) n_groups *= 2;
  hipLaunchKernelGGL(filter_backprop_1x1_f16_reduce_kernel,
                     dim3(vecs / (256 / n_groups)), dim3(256), 0, stream,
                     reinterpret_cast<const float4v*>(part), dw, n_tiles,
                     g.c_tiles, g.n_splits, n_groups, plan.a, plan.b,
                     p.features);
  return SNN_HIP_OK;
}

}  // namespace snn
