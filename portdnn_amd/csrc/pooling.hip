// Max / average pooling for gfx950: bandwidth-bound kernels, no MFMA.
// Stand-ins for portDNN's PoolingOp functors (src/pooling/kernels.h:43-414)
// with the operators of src/pooling/operators_impl.h:27-113.
//
// Forward: one lane per output channel vector (4 channels when C % 4 == 0, as
// src/pooling/launch_pooling.cc:134-143 chooses), channel index fastest, so a
// wave reads contiguous NHWC runs.  The window is clipped to the image;
// average divides by the clipped element count.
#include <cfloat>

#include <cstdlib>

#include "gemm_tile.h"
#include "snn_kernels.h"

namespace snn {
namespace {

// numeric_limits<T>::lowest(), the start value of the max operators.
template <typename T>
__device__ constexpr float lowest_of();
template <>
__device__ constexpr float lowest_of<float>() { return -FLT_MAX; }
template <>
__device__ constexpr float lowest_of<_Float16>() { return -65504.f; }

// Accumulators with portDNN's semantics.
struct MaxOp {
  float v;
  __device__ void init(float lowest) { v = lowest; }
  __device__ void accumulate(float x) {
    if (x > v) v = x;  // a NaN never compares greater
  }
  __device__ void merge(float partial) { accumulate(partial); }
  __device__ float value(int) const { return v; }
};
struct MaxNanOp {
  float v;
  __device__ void init(float lowest) { v = lowest; }
  __device__ void accumulate(float x) {
    if (x != x || x > v) v = x;  // a NaN wins and then sticks
  }
  __device__ void merge(float partial) { accumulate(partial); }
  __device__ float value(int) const { return v; }
};
struct AvgOp {
  float v;
  __device__ void init(float) { v = 0.f; }
  __device__ void accumulate(float x) { v += x; }
  __device__ void merge(float partial) { v += partial; }
  __device__ float value(int tally) const {
    return v / static_cast<float>(tally);
  }
};

template <typename T, int VEC>
struct VecIO;
template <>
struct VecIO<float, 1> {
  __device__ static void load(const float* p, float (&v)[1]) { v[0] = *p; }
  __device__ static void store(float* p, const float (&v)[1]) { *p = v[0]; }
};
template <>
struct VecIO<float, 4> {
  __device__ static void load(const float* p, float (&v)[4]) {
    const float4 t = *reinterpret_cast<const float4*>(p);
    v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
  }
  __device__ static void store(float* p, const float (&v)[4]) {
    *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
  }
};
template <>
struct VecIO<_Float16, 1> {
  __device__ static void load(const _Float16* p, float (&v)[1]) {
    v[0] = static_cast<float>(*p);
  }
  __device__ static void store(_Float16* p, const float (&v)[1]) {
    *p = static_cast<_Float16>(v[0]);
  }
};
template <>
struct VecIO<_Float16, 4> {
  typedef _Float16 half4 __attribute__((ext_vector_type(4)));
  __device__ static void load(const _Float16* p, float (&v)[4]) {
    const half4 t = *reinterpret_cast<const half4*>(p);
    v[0] = static_cast<float>(t.x); v[1] = static_cast<float>(t.y);
    v[2] = static_cast<float>(t.z); v[3] = static_cast<float>(t.w);
  }
  __device__ static void store(_Float16* p, const float (&v)[4]) {
    half4 t;
    t.x = static_cast<_Float16>(v[0]); t.y = static_cast<_Float16>(v[1]);
    t.z = static_cast<_Float16>(v[2]); t.w = static_cast<_Float16>(v[3]);
    *reinterpret_cast<half4*>(p) = t;
  }
};

template <typename T, typename Op, int VEC>
__global__ void __launch_bounds__(256)
    pool_forward_kernel(const T* __restrict__ in, T* __restrict__ out,
                        snn_hip_pooling_params p, size_t n_vec) {
  const size_t idx = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (idx >= n_vec) return;
  const int C = p.channels;
  const int cv = C / VEC;
  const int c = static_cast<int>(idx % cv) * VEC;
  size_t pix = idx / cv;
  const int ox = static_cast<int>(pix % p.out_cols);
  pix /= p.out_cols;
  const int oy = static_cast<int>(pix % p.out_rows);
  const int n = static_cast<int>(pix / p.out_rows);
  int r0 = oy * p.stride_rows - p.pad_rows;
  const int r1 = min(r0 + p.window_rows, p.in_rows);
  r0 = max(r0, 0);
  int c0 = ox * p.stride_cols - p.pad_cols;
  const int c1 = min(c0 + p.window_cols, p.in_cols);
  c0 = max(c0, 0);
  const T* in_n = in + static_cast<size_t>(n) * p.in_rows * p.in_cols * C + c;
  Op op[VEC];
#pragma unroll
  for (int i = 0; i < VEC; ++i) op[i].init(lowest_of<T>());
  for (int r = r0; r < r1; ++r) {
    for (int col = c0; col < c1; ++col) {
      float v[VEC];
      VecIO<T, VEC>::load(in_n + (static_cast<size_t>(r) * p.in_cols + col) * C,
                          v);
#pragma unroll
      for (int i = 0; i < VEC; ++i) op[i].accumulate(v[i]);
    }
  }
  // the number of elements accumulated (src/pooling/operators_impl.h:61-82
  // counts them one by one): none when the window misses the image on an axis
  const int tally = max(r1 - r0, 0) * max(c1 - c0, 0);
  float res[VEC];
#pragma unroll
  for (int i = 0; i < VEC; ++i) res[i] = op[i].value(tally);
  VecIO<T, VEC>::store(out + idx * VEC, res);
}

// ---- 3x3 forward, four channels per lane, TH consecutive output rows -------
// Each input row of the strip is loaded once (three column taps) and folded
// into every output row it belongs to, so vertically adjacent windows share
// their rows in registers.  Taps outside the image are redirected to the
// nearest in-image tap of the same window for the max operators (a duplicate
// does not change a maximum, nor whether a NaN is present) and read as zero
// for the average, whose divisor is the analytic in-bounds count.
typedef unsigned int uint4v __attribute__((ext_vector_type(4)));
typedef unsigned int uint2v __attribute__((ext_vector_type(2)));
constexpr unsigned kOobOffset = 0x7FFFFFF0u;
// Cache policy bits of the input loads (0 = default; a build-time switch for
// experiments, e.g. -DSNN_MEM_LOAD_AUX=2 for streaming loads).
#ifndef SNN_MEM_LOAD_AUX
#define SNN_MEM_LOAD_AUX 0
#endif

__device__ inline __amdgpu_buffer_rsrc_t make_rsrc(const void* p, size_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0,
                                           static_cast<unsigned>(bytes),
                                           0x00020000);
}
template <typename T>
struct BufVec4;
template <>
struct BufVec4<float> {
  __device__ static void load(__amdgpu_buffer_rsrc_t r, unsigned off,
                              float (&v)[4]) {
    const float4 t = __builtin_bit_cast(
        float4, __builtin_amdgcn_raw_buffer_load_b128(r, off, 0, SNN_MEM_LOAD_AUX));
    v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
  }
  __device__ static void store(__amdgpu_buffer_rsrc_t r, unsigned off,
                               const float (&v)[4]) {
    __builtin_amdgcn_raw_buffer_store_b128(
        __builtin_bit_cast(uint4v, make_float4(v[0], v[1], v[2], v[3])), r, off,
        0, 2);  // streaming store
  }
};
template <>
struct BufVec4<_Float16> {
  typedef _Float16 half4 __attribute__((ext_vector_type(4)));
  __device__ static void load(__amdgpu_buffer_rsrc_t r, unsigned off,
                              float (&v)[4]) {
    const half4 t = __builtin_bit_cast(
        half4, __builtin_amdgcn_raw_buffer_load_b64(r, off, 0, SNN_MEM_LOAD_AUX));
    v[0] = static_cast<float>(t.x); v[1] = static_cast<float>(t.y);
    v[2] = static_cast<float>(t.z); v[3] = static_cast<float>(t.w);
  }
  __device__ static void store(__amdgpu_buffer_rsrc_t r, unsigned off,
                               const float (&v)[4]) {
    half4 t;
    t.x = static_cast<_Float16>(v[0]); t.y = static_cast<_Float16>(v[1]);
    t.z = static_cast<_Float16>(v[2]); t.w = static_cast<_Float16>(v[3]);
    __builtin_amdgcn_raw_buffer_store_b64(__builtin_bit_cast(uint2v, t), r, off,
                                          0, 2);
  }
};

template <typename Op>
struct IsAverage {
  static constexpr bool value = false;
};
template <>
struct IsAverage<AvgOp> {
  static constexpr bool value = true;
};

template <typename T, typename Op, int STRIDE, int TH>
__global__ void __launch_bounds__(256)
    pool_forward_3x3_strip_kernel(const T* __restrict__ in, T* __restrict__ out,
                                  snn_hip_pooling_params p, int n_strips,
                                  unsigned n_items) {
  // Work-groups go round-robin to the 8 XCDs; the remap gives every XCD one
  // contiguous run of the index space, so vertically adjacent strips (which
  // share an input row at stride 2, two at stride 1) meet in the same L2.
  const unsigned idx =
      gemm::xcd_remap(blockIdx.x, gridDim.x) * 256u + threadIdx.x;
  if (idx >= n_items) return;
  const int C = p.channels;
  const unsigned cv = static_cast<unsigned>(C) / 4u;
  const int c = static_cast<int>(idx % cv) * 4;
  unsigned rest = idx / cv;
  const int ox = static_cast<int>(rest % static_cast<unsigned>(p.out_cols));
  rest /= static_cast<unsigned>(p.out_cols);
  const int strip = static_cast<int>(rest % static_cast<unsigned>(n_strips));
  const int n = static_cast<int>(rest / static_cast<unsigned>(n_strips));
  const int oy0 = strip * TH;
  constexpr unsigned kEsz = sizeof(T);
  constexpr bool kAvg = IsAverage<Op>::value;
  const __amdgpu_buffer_rsrc_t in_rsrc = make_rsrc(
      in, static_cast<size_t>(p.batch) * p.in_rows * p.in_cols * C * kEsz);
  const __amdgpu_buffer_rsrc_t out_rsrc = make_rsrc(
      out, static_cast<size_t>(p.batch) * p.out_rows * p.out_cols * C * kEsz);
  Op acc[TH][4];
#pragma unroll
  for (int t = 0; t < TH; ++t)
#pragma unroll
    for (int i = 0; i < 4; ++i) acc[t][i].init(lowest_of<T>());
  const int x0 = ox * STRIDE - p.pad_cols;
  const int y0 = oy0 * STRIDE - p.pad_rows;
  const int img = n * p.in_rows * p.in_cols;
  // column taps: clamp into the image (max) or mark as zero fill (average)
  int col[3];
  bool col_ok[3];
#pragma unroll
  for (int sx = 0; sx < 3; ++sx) {
    col_ok[sx] = static_cast<unsigned>(x0 + sx) < static_cast<unsigned>(p.in_cols);
    col[sx] = min(max(x0 + sx, 0), p.in_cols - 1);
  }
  constexpr int NR = (TH - 1) * STRIDE + 3;
#pragma unroll
  for (int j = 0; j < NR; ++j) {
    const int y = y0 + j;
    const bool row_ok = static_cast<unsigned>(y) < static_cast<unsigned>(p.in_rows);
    // For the max operators a row below / above the image is replaced by the
    // nearest image row of the same window; rows that belong to no window of
    // this strip are never folded in.
    const int yc = min(max(y, 0), p.in_rows - 1);
    float row[3][4];
#pragma unroll
    for (int sx = 0; sx < 3; ++sx) {
      unsigned off;
      if (kAvg) {
        off = (row_ok & col_ok[sx])
                  ? static_cast<unsigned>((img + y * p.in_cols + x0 + sx) * C + c) * kEsz
                  : kOobOffset;
      } else {
        off = static_cast<unsigned>((img + yc * p.in_cols + col[sx]) * C + c) * kEsz;
      }
      BufVec4<T>::load(in_rsrc, off, row[sx]);
    }
#pragma unroll
    for (int t = 0; t < TH; ++t) {
      const int r = j - t * STRIDE;
      if (r < 0 || r > 2) continue;
#pragma unroll
      for (int sx = 0; sx < 3; ++sx)
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[t][i].accumulate(row[sx][i]);
    }
  }
  const int c_lo = max(x0, 0), c_hi = min(x0 + 3, p.in_cols);
  const int out_base = ((n * p.out_rows + oy0) * p.out_cols + ox) * C + c;
#pragma unroll
  for (int t = 0; t < TH; ++t) {
    const int ry = y0 + t * STRIDE;
    const int tally = (min(ry + 3, p.in_rows) - max(ry, 0)) * (c_hi - c_lo);
    float res[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) res[i] = acc[t][i].value(tally);
    BufVec4<T>::store(out_rsrc,
                      oy0 + t < p.out_rows
                          ? static_cast<unsigned>(out_base + t * p.out_cols * C) * kEsz
                          : kOobOffset,
                      res);
  }
}

// ---- 3x3 stride-2 forward, fp32, tall strips --------------------------------
// C = 4 * CV with CV in {8, 16, 32}.  A wave is 64 / CV pixel lanes x CV
// channel vectors; a lane owns one output pixel, i.e. the first two columns of
// its window, loads only those, and takes the third column -- the first
// column of the pixel lane to its right -- with a cross-lane read
// (ds_bpermute: the LDS crossbar, no LDS memory).  Only the last pixel lane of
// a wave loads that column itself.  A strip is TH output rows tall: it walks
// down 2 TH + 1 input rows with two rows of open windows and stores an output
// row as soon as its third window row has been folded in, so two strips share
// one input row in 2 TH + 1.  Rows the strip owns are read with streaming
// loads, the shared row and the wave-edge column with ordinary ones;
// work-groups are not remapped to XCDs, so consecutive groups stream
// consecutive runs of the tensor on all XCDs together.  Taps outside the
// image never enter a maximum (they are replaced by lowest()) and read as
// zero for the average, whose divisor is the in-image element count; the
// window is scanned row-major as in src/pooling/kernels.h:61-99.
template <typename Op, int TH, int CV>
__global__ void __launch_bounds__(256)
    pool_forward_3x3_s2_tall_kernel(const float* __restrict__ in,
                                    float* __restrict__ out,
                                    snn_hip_pooling_params p, int n_strips,
                                    int n_wcols, unsigned n_waves) {
  constexpr int PXW = 64 / CV;
  constexpr int NR = 2 * TH + 1;
  constexpr bool kAvg = IsAverage<Op>::value;
  constexpr int kNt = 2;  // streaming (nt) load
  const unsigned w = blockIdx.x * 4u + (threadIdx.x >> 6);
  if (w >= n_waves) return;  // whole waves only (cross-lane reads below)
  const int lane = threadIdx.x & 63;
  const int cvi = lane % CV, pl = lane / CV;
  const int wcol = static_cast<int>(w % static_cast<unsigned>(n_wcols));
  const unsigned rest = w / static_cast<unsigned>(n_wcols);
  const int strip = static_cast<int>(rest % static_cast<unsigned>(n_strips));
  const int n = static_cast<int>(rest / static_cast<unsigned>(n_strips));
  const int C = p.channels, c = cvi * 4;
  const __amdgpu_buffer_rsrc_t in_rsrc = make_rsrc(
      in, static_cast<size_t>(p.batch) * p.in_rows * p.in_cols * C * 4);
  const __amdgpu_buffer_rsrc_t out_rsrc = make_rsrc(
      out, static_cast<size_t>(p.batch) * p.out_rows * p.out_cols * C * 4);
  const float ident = kAvg ? 0.f : lowest_of<float>();
  const int oy0 = strip * TH;
  const int ox = wcol * PXW + pl;
  const int col0 = 2 * ox - p.pad_cols;   // first window column
  const int y0 = 2 * oy0 - p.pad_rows;    // first input row of the strip
  const int xr = 2 * (wcol + 1) * PXW - p.pad_cols;  // the wave's halo column
  const bool last = pl == PXW - 1;
  const bool c0_ok =
      static_cast<unsigned>(col0) < static_cast<unsigned>(p.in_cols);
  const bool c1_ok =
      static_cast<unsigned>(col0 + 1) < static_cast<unsigned>(p.in_cols);
  const bool r_ok =
      last && static_cast<unsigned>(xr) < static_cast<unsigned>(p.in_cols);
  const int row0 = (n * p.in_rows + y0) * p.in_cols * C + c;
  const int rstride = p.in_cols * C;
  const int src_r = (lane + CV) * 4;

  float own[NR][2][4], hr[NR][4];
#pragma unroll
  for (int j = 0; j < NR; ++j) {
    const bool row_ok =
        static_cast<unsigned>(y0 + j) < static_cast<unsigned>(p.in_rows);
    const bool mine = j < 2 * TH;  // the last row also opens the next strip
#pragma unroll
    for (int k = 0; k < 2; ++k) {
      const bool ok = row_ok && (k == 0 ? c0_ok : c1_ok);
      const unsigned off =
          ok ? static_cast<unsigned>(row0 + j * rstride + (col0 + k) * C) * 4u
             : kOobOffset;
      const float4 t = __builtin_bit_cast(
          float4, mine ? __builtin_amdgcn_raw_buffer_load_b128(in_rsrc, off, 0,
                                                               kNt)
                       : __builtin_amdgcn_raw_buffer_load_b128(in_rsrc, off, 0,
                                                               0));
      own[j][k][0] = ok ? t.x : ident; own[j][k][1] = ok ? t.y : ident;
      own[j][k][2] = ok ? t.z : ident; own[j][k][3] = ok ? t.w : ident;
    }
    const bool ok = row_ok && r_ok;
    const float4 t = __builtin_bit_cast(
        float4,
        __builtin_amdgcn_raw_buffer_load_b128(
            in_rsrc,
            ok ? static_cast<unsigned>(row0 + j * rstride + xr * C) * 4u
               : kOobOffset,
            0, 0));
    hr[j][0] = ok ? t.x : ident; hr[j][1] = ok ? t.y : ident;
    hr[j][2] = ok ? t.z : ident; hr[j][3] = ok ? t.w : ident;
  }

  const int c_lo = max(col0, 0), c_hi = min(col0 + 3, p.in_cols);
  Op acc[2][4];
#pragma unroll
  for (int j = 0; j < NR; ++j) {
    float third[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float from_right = __builtin_bit_cast(
          float, __builtin_amdgcn_ds_bpermute(
                     src_r, __builtin_bit_cast(int, own[j][0][i])));
      third[i] = last ? hr[j][i] : from_right;
    }
    // input row j is window row r of output row t = (j - r) / 2; the older
    // output row first
#pragma unroll
    for (int r = 2; r >= 0; r -= 2) {
      if (j - r < 0 || ((j - r) & 1) != 0) continue;
      const int t = (j - r) / 2;
      if (t >= TH) continue;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        if (r == 0) acc[t & 1][i].init(lowest_of<float>());
        acc[t & 1][i].accumulate(own[j][0][i]);
        acc[t & 1][i].accumulate(own[j][1][i]);
        acc[t & 1][i].accumulate(third[i]);
      }
      if (r == 2) {
        const int ry = y0 + 2 * t;
        const int tally = max(min(ry + 3, p.in_rows) - max(ry, 0), 0) *
                          max(c_hi - c_lo, 0);
        float res[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) res[i] = acc[t & 1][i].value(tally);
        const bool ok = oy0 + t < p.out_rows && ox < p.out_cols;
        BufVec4<float>::store(
            out_rsrc,
            ok ? static_cast<unsigned>(
                     ((n * p.out_rows + oy0 + t) * p.out_cols + ox) * C + c) * 4u
               : kOobOffset,
            res);
      }
    }
    // odd input rows are window row 1 of one output row only
    if ((j & 1) != 0) {
      const int t = (j - 1) / 2;
      if (t < TH) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          acc[t & 1][i].accumulate(own[j][0][i]);
          acc[t & 1][i].accumulate(own[j][1][i]);
          acc[t & 1][i].accumulate(third[i]);
        }
      }
    }
  }
}

// ---- windows covering most of a small image (global pooling) ---------------
// One work-group per (image, output pixel, group of 16 channel vectors).  The
// window taps are dealt to 16 tap slices -- four per wave, lane = slice * 16 +
// channel vector -- so the 49 taps of a 7x7 global average are at most four
// independent 16-byte loads per lane, all in flight together, and 16 lanes
// read one contiguous 256-byte run of a pixel's channels.  The slices of a
// wave are combined with two cross-lane exchanges (no LDS memory), the four
// waves through 1 KiB of LDS.
template <typename T, typename Op>
__global__ void __launch_bounds__(256)
    pool_forward_tapsplit_kernel(const T* __restrict__ in, T* __restrict__ out,
                                 snn_hip_pooling_params p, int n_groups) {
  __shared__ float part[4][16][4];
  const int C = p.channels;
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int cvl = lane & 15;
  const int slice = wave * 4 + (lane >> 4);  // 0 .. 15
  unsigned b = blockIdx.x;
  const int grp = static_cast<int>(b % static_cast<unsigned>(n_groups));
  b /= static_cast<unsigned>(n_groups);
  const int ox = static_cast<int>(b % static_cast<unsigned>(p.out_cols));
  b /= static_cast<unsigned>(p.out_cols);
  const int oy = static_cast<int>(b % static_cast<unsigned>(p.out_rows));
  const int n = static_cast<int>(b / static_cast<unsigned>(p.out_rows));
  const int c = (grp * 16 + cvl) * 4;
  const bool active = c < C;
  int r0 = oy * p.stride_rows - p.pad_rows;
  const int r1 = min(r0 + p.window_rows, p.in_rows);
  r0 = max(r0, 0);
  int c0 = ox * p.stride_cols - p.pad_cols;
  const int c1 = min(c0 + p.window_cols, p.in_cols);
  c0 = max(c0, 0);
  // a window wholly outside the image on an axis has no taps (both extents
  // negative must not multiply to a positive count)
  const int width = max(c1 - c0, 0);
  const int n_taps = max(r1 - r0, 0) * width;
  Op acc[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) acc[i].init(lowest_of<T>());
  if (active && n_taps > 0) {
    const T* base =
        in + static_cast<size_t>(n) * p.in_rows * p.in_cols * C + c;
    for (int t0 = slice; t0 < n_taps; t0 += 64) {
      float v[4][4];
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        // a tap index past the end re-reads the last tap and is not counted
        const int t = min(t0 + 16 * k, n_taps - 1);
        const int r = r0 + t / width, col = c0 + t % width;
        VecIO<T, 4>::load(base + (static_cast<size_t>(r) * p.in_cols + col) * C,
                          v[k]);
      }
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        if (t0 + 16 * k < n_taps) {
#pragma unroll
          for (int i = 0; i < 4; ++i) acc[i].accumulate(v[k][i]);
        }
      }
    }
  }
  // the four tap slices of this wave: lanes l, l ^ 16, l ^ 32, l ^ 48
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    acc[i].merge(__shfl_xor(acc[i].v, 16));
    acc[i].merge(__shfl_xor(acc[i].v, 32));
  }
  if (lane < 16) {
#pragma unroll
    for (int i = 0; i < 4; ++i) part[wave][lane][i] = acc[i].v;
  }
  __syncthreads();
  if (wave == 0 && lane < 16 && active) {
    float res[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      Op total = acc[i];
      for (int w = 1; w < 4; ++w) total.merge(part[w][lane][i]);
      res[i] = total.value(n_taps);
    }
    VecIO<T, 4>::store(
        out + ((static_cast<size_t>(n) * p.out_rows + oy) * p.out_cols + ox) * C +
            c,
        res);
  }
}

__device__ inline bool pool_equal(float a, float b, bool nan_mode) {
  return a == b || (nan_mode && a != a && b != b);
}

// Max gradient: one lane per input element.  For every output whose window
// covers this element and whose value equals it, the gradient is taken only if
// no earlier element of that window (row-major) also equals the output -- the
// first maximum wins (src/pooling/kernels.h:141-239).
template <int VEC>
struct GradVec;
template <>
struct GradVec<1> {
  __device__ static void load(const float* p, float (&v)[1]) { v[0] = *p; }
  __device__ static void store(float* p, const float (&v)[1]) { *p = v[0]; }
  __device__ static void load(const _Float16* p, float (&v)[1]) {
    v[0] = static_cast<float>(*p);
  }
  __device__ static void store(_Float16* p, const float (&v)[1]) {
    *p = static_cast<_Float16>(v[0]);
  }
};
template <>
struct GradVec<4> {
  typedef _Float16 half4 __attribute__((ext_vector_type(4)));
  __device__ static void load(const float* p, float (&v)[4]) {
    const float4 t = *reinterpret_cast<const float4*>(p);
    v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
  }
  __device__ static void store(float* p, const float (&v)[4]) {
    *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
  }
  __device__ static void load(const _Float16* p, float (&v)[4]) {
    const half4 t = *reinterpret_cast<const half4*>(p);
    v[0] = static_cast<float>(t.x); v[1] = static_cast<float>(t.y);
    v[2] = static_cast<float>(t.z); v[3] = static_cast<float>(t.w);
  }
  __device__ static void store(_Float16* p, const float (&v)[4]) {
    half4 t;
    t.x = static_cast<_Float16>(v[0]); t.y = static_cast<_Float16>(v[1]);
    t.z = static_cast<_Float16>(v[2]); t.w = static_cast<_Float16>(v[3]);
    *reinterpret_cast<half4*>(p) = t;
  }
};

// VEC channels per lane (4 when the channel count and the pointers allow
// 16-byte accesses).
template <int VEC, typename T = float>
__global__ void __launch_bounds__(256)
    pool_max_grad_kernel(const T* __restrict__ in, const T* __restrict__ out,
                         const T* __restrict__ dy, T* __restrict__ dx,
                         snn_hip_pooling_params p, bool nan_mode, size_t n_vec) {
  const size_t idx = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (idx >= n_vec) return;
  const int C = p.channels;
  const int cv = C / VEC;
  const int ch = static_cast<int>(idx % cv) * VEC;
  size_t pix = idx / cv;
  const int x = static_cast<int>(pix % p.in_cols);
  pix /= p.in_cols;
  const int y = static_cast<int>(pix % p.in_rows);
  const int n = static_cast<int>(pix / p.in_rows);
  float mine[VEC];
  GradVec<VEC>::load(in + idx * VEC, mine);
  const T* in_n = in + static_cast<size_t>(n) * p.in_rows * p.in_cols * C + ch;
  const size_t out_base =
      static_cast<size_t>(n) * p.out_rows * p.out_cols * C + ch;
  // outputs whose (unclipped) window contains y / x
  const int py = y + p.pad_rows, px = x + p.pad_cols;
  const int oy_begin =
      py < p.window_rows ? 0 : (py - p.window_rows) / p.stride_rows + 1;
  const int oy_end = min(py / p.stride_rows + 1, p.out_rows);
  const int ox_begin =
      px < p.window_cols ? 0 : (px - p.window_cols) / p.stride_cols + 1;
  const int ox_end = min(px / p.stride_cols + 1, p.out_cols);
  float grad[VEC];
#pragma unroll
  for (int i = 0; i < VEC; ++i) grad[i] = 0.f;
  for (int oy = oy_begin; oy < oy_end; ++oy) {
    int r0 = oy * p.stride_rows - p.pad_rows;
    const int r1 = min(r0 + p.window_rows, p.in_rows);
    r0 = max(r0, 0);
    for (int ox = ox_begin; ox < ox_end; ++ox) {
      int c0 = ox * p.stride_cols - p.pad_cols;
      const int c1 = min(c0 + p.window_cols, p.in_cols);
      c0 = max(c0, 0);
      const size_t o = out_base + (static_cast<size_t>(oy) * p.out_cols + ox) * C;
      float target[VEC];
      GradVec<VEC>::load(out + o, target);
      // components of this lane that equal the window's maximum and have not
      // yet been ruled out by an earlier equal element
      bool live[VEC];
      bool any = false;
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        live[i] = pool_equal(mine[i], target[i], nan_mode);
        any |= live[i];
      }
      if (!any) continue;
      bool reached = false;
      for (int r = r0; r < r1 && any && !reached; ++r) {
        for (int col = c0; col < c1; ++col) {
          if (r == y && col == x) {
            reached = true;  // nothing earlier matched for the live components
            break;
          }
          float v[VEC];
          GradVec<VEC>::load(
              in_n + (static_cast<size_t>(r) * p.in_cols + col) * C, v);
          any = false;
#pragma unroll
          for (int i = 0; i < VEC; ++i) {
            live[i] = live[i] && !pool_equal(v[i], target[i], nan_mode);
            any |= live[i];
          }
          if (!any) break;
        }
      }
      if (!any) continue;
      float g[VEC];
      GradVec<VEC>::load(dy + o, g);
#pragma unroll
      for (int i = 0; i < VEC; ++i)
        if (live[i]) grad[i] += g[i];
    }
  }
  GradVec<VEC>::store(dx + idx * VEC, grad);
}

// Average gradient: every covering output contributes dY / clipped window
// size (src/pooling/kernels.h:291-414).
template <int VEC, typename T = float>
__global__ void __launch_bounds__(256)
    pool_avg_grad_kernel(const T* __restrict__ dy, T* __restrict__ dx,
                         snn_hip_pooling_params p, size_t n_vec) {
  const size_t idx = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (idx >= n_vec) return;
  const int C = p.channels;
  const int cv = C / VEC;
  const int ch = static_cast<int>(idx % cv) * VEC;
  size_t pix = idx / cv;
  const int x = static_cast<int>(pix % p.in_cols);
  pix /= p.in_cols;
  const int y = static_cast<int>(pix % p.in_rows);
  const int n = static_cast<int>(pix / p.in_rows);
  const size_t out_base =
      static_cast<size_t>(n) * p.out_rows * p.out_cols * C + ch;
  const int py = y + p.pad_rows, px = x + p.pad_cols;
  const int oy_begin =
      py < p.window_rows ? 0 : (py - p.window_rows) / p.stride_rows + 1;
  const int oy_end = min(py / p.stride_rows + 1, p.out_rows);
  const int ox_begin =
      px < p.window_cols ? 0 : (px - p.window_cols) / p.stride_cols + 1;
  const int ox_end = min(px / p.stride_cols + 1, p.out_cols);
  float grad[VEC];
#pragma unroll
  for (int i = 0; i < VEC; ++i) grad[i] = 0.f;
  for (int oy = oy_begin; oy < oy_end; ++oy) {
    int r0 = oy * p.stride_rows - p.pad_rows;
    const int r1 = min(r0 + p.window_rows, p.in_rows);
    r0 = max(r0, 0);
    for (int ox = ox_begin; ox < ox_end; ++ox) {
      int c0 = ox * p.stride_cols - p.pad_cols;
      const int c1 = min(c0 + p.window_cols, p.in_cols);
      c0 = max(c0, 0);
      const float count = static_cast<float>((r1 - r0) * (c1 - c0));
      float g[VEC];
      GradVec<VEC>::load(
          dy + out_base + (static_cast<size_t>(oy) * p.out_cols + ox) * C, g);
#pragma unroll
      for (int i = 0; i < VEC; ++i) grad[i] += g[i] / count;
    }
  }
  GradVec<VEC>::store(dx + idx * VEC, grad);
}

// The same gradient with TH consecutive input rows of one column per lane
// (four channels): the index arithmetic and the column range are computed once
// per strip, and every contributing dY / count is formed once and added to
// each of the strip's rows its window covers, in the same output-row,
// output-column order as above.
template <int TH>
__global__ void __launch_bounds__(256)
    pool_avg_grad_strip_kernel(const float* __restrict__ dy,
                               float* __restrict__ dx, snn_hip_pooling_params p,
                               int n_strips, unsigned n_items) {
  const unsigned idx = blockIdx.x * 256u + threadIdx.x;
  if (idx >= n_items) return;
  const int C = p.channels;
  const unsigned cv = static_cast<unsigned>(C) / 4u;
  const int ch = static_cast<int>(idx % cv) * 4;
  unsigned t = idx / cv;
  const int x = static_cast<int>(t % static_cast<unsigned>(p.in_cols));
  t /= static_cast<unsigned>(p.in_cols);
  const int y0 = static_cast<int>(t % static_cast<unsigned>(n_strips)) * TH;
  const int n = static_cast<int>(t / static_cast<unsigned>(n_strips));
  const int y_last = min(y0 + TH, p.in_rows) - 1;
  const int px = x + p.pad_cols;
  const int ox_begin =
      px < p.window_cols ? 0 : (px - p.window_cols) / p.stride_cols + 1;
  const int ox_end = min(px / p.stride_cols + 1, p.out_cols);
  const int py0 = y0 + p.pad_rows;
  const int oy_begin =
      py0 < p.window_rows ? 0 : (py0 - p.window_rows) / p.stride_rows + 1;
  const int oy_end = min((y_last + p.pad_rows) / p.stride_rows + 1, p.out_rows);
  const float* dy_n =
      dy + static_cast<size_t>(n) * p.out_rows * p.out_cols * C + ch;
  float grad[TH][4];
#pragma unroll
  for (int i = 0; i < TH; ++i)
#pragma unroll
    for (int e = 0; e < 4; ++e) grad[i][e] = 0.f;
  for (int oy = oy_begin; oy < oy_end; ++oy) {
    int r0 = oy * p.stride_rows - p.pad_rows;
    const int r1 = min(r0 + p.window_rows, p.in_rows);
    r0 = max(r0, 0);
    for (int ox = ox_begin; ox < ox_end; ++ox) {
      int c0 = ox * p.stride_cols - p.pad_cols;
      const int c1 = min(c0 + p.window_cols, p.in_cols);
      c0 = max(c0, 0);
      const float count = static_cast<float>((r1 - r0) * (c1 - c0));
      float g[4];
      GradVec<4>::load(dy_n + (static_cast<size_t>(oy) * p.out_cols + ox) * C,
                       g);
#pragma unroll
      for (int e = 0; e < 4; ++e) g[e] = g[e] / count;
#pragma unroll
      for (int i = 0; i < TH; ++i) {
        if (y0 + i >= r0 && y0 + i < r1) {
#pragma unroll
          for (int e = 0; e < 4; ++e) grad[i][e] += g[e];
        }
      }
    }
  }
  float* dx_p =
      dx + ((static_cast<size_t>(n) * p.in_rows + y0) * p.in_cols + x) * C + ch;
  const size_t row_elems = static_cast<size_t>(p.in_cols) * C;
#pragma unroll
  for (int i = 0; i < TH; ++i)
    if (y0 + i <= y_last) GradVec<4>::store(dx_p + i * row_elems, grad[i]);
}

// The average gradient for 3x3 windows at stride 2 (no LDS, all loads of a
// block row issued together).  In padded coordinates an input pixel with an
// even row lies in the last row of window row (row / 2 - 1) and the first of
// (row / 2), one with an odd row only in the middle of (row / 2); columns
// alike.  So the 2x2 input pixels of block (br, bc) take their gradient from
// the windows (br - 1 .. br) x (bc - 1 .. bc) only: a lane walks TH block rows
// of one block column, loads the two dY vectors of a window row once, divides
// them by the windows' in-image element counts and carries them down as the
// next block row's "windows above".  The terms are added in the reference's
// order (window row, then window column, starting from zero;
// src/pooling/kernels.h:291-375); a window that does not exist contributes
// +0, which leaves every sum as it is.
template <int TH, typename T = float>
__global__ void __launch_bounds__(256)
    pool_avg_grad_3x3_s2_kernel(const T* __restrict__ dy,
                                T* __restrict__ dx,
                                snn_hip_pooling_params p, int n_bcols,
                                int n_strips, unsigned n_items) {
  const unsigned idx = blockIdx.x * 256u + threadIdx.x;
  if (idx >= n_items) return;
  const int C = p.channels;
  const unsigned cv = static_cast<unsigned>(C) / 4u;
  const int ch = static_cast<int>(idx % cv) * 4;
  unsigned t = idx / cv;
  const int bc = static_cast<int>(t % static_cast<unsigned>(n_bcols)) +
                 p.pad_cols / 2;
  t /= static_cast<unsigned>(n_bcols);
  const int br0 = static_cast<int>(t % static_cast<unsigned>(n_strips)) * TH +
                  p.pad_rows / 2;
  const int n = static_cast<int>(t / static_cast<unsigned>(n_strips));
  constexpr unsigned kEsz = sizeof(T);
  const size_t in_elems =
      static_cast<size_t>(p.batch) * p.in_rows * p.in_cols * C;
  const size_t out_elems =
      static_cast<size_t>(p.batch) * p.out_rows * p.out_cols * C;
  const __amdgpu_buffer_rsrc_t dy_rsrc = make_rsrc(dy, out_elems * kEsz);
  const __amdgpu_buffer_rsrc_t dx_rsrc = make_rsrc(dx, in_elems * kEsz);

  // windows bc - 1 and bc: present, and their number of in-image columns
  bool w_ok[2];
  int w_cols[2];
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int ox = bc - 1 + j;
    w_ok[j] = static_cast<unsigned>(ox) < static_cast<unsigned>(p.out_cols);
    const int c0 = 2 * ox - p.pad_cols;
    w_cols[j] = max(min(c0 + 3, p.in_cols) - max(c0, 0), 1);
  }
  // dY[oy][bc - 1 .. bc] / count, zeros for windows that do not exist
  auto load_row = [&](int oy, float (&g)[2][4]) {
    const bool row_ok =
        static_cast<unsigned>(oy) < static_cast<unsigned>(p.out_rows);
    const unsigned base =
        static_cast<unsigned>(((n * p.out_rows + oy) * p.out_cols + bc - 1) *
                                  C + ch) * kEsz;
#pragma unroll
    for (int j = 0; j < 2; ++j)
      BufVec4<T>::load(dy_rsrc,
                           (row_ok && w_ok[j])
                               ? base + static_cast<unsigned>(j * C) * kEsz
                               : kOobOffset,
                           g[j]);
  };
  auto divide_row = [&](int oy, float (&g)[2][4]) {
    const int r0 = 2 * oy - p.pad_rows;
    const int w_rows = max(min(r0 + 3, p.in_rows) - max(r0, 0), 1);
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const float count = static_cast<float>(w_rows * w_cols[j]);
#pragma unroll
      for (int e = 0; e < 4; ++e) g[j][e] = g[j][e] / count;
    }
  };
  const int x0 = 2 * bc - p.pad_cols;
  const bool x_ok[2] = {
      static_cast<unsigned>(x0) < static_cast<unsigned>(p.in_cols),
      static_cast<unsigned>(x0 + 1) < static_cast<unsigned>(p.in_cols)};
  const unsigned row_bytes = static_cast<unsigned>(p.in_cols * C) * kEsz;
  const unsigned col_bytes = static_cast<unsigned>(C) * kEsz;

  float rows[TH + 1][2][4];
#pragma unroll
  for (int i = 0; i <= TH; ++i) load_row(br0 - 1 + i, rows[i]);
#pragma unroll
  for (int i = 0; i <= TH; ++i) divide_row(br0 - 1 + i, rows[i]);
#pragma unroll
  for (int i = 0; i < TH; ++i) {
    const int br = br0 + i;
    const float (&above)[2][4] = rows[i];
    const float (&here)[2][4] = rows[i + 1];
    float ee[4], eo[4], oe[4], oo[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      ee[e] = (((0.f + above[0][e]) + above[1][e]) + here[0][e]) + here[1][e];
      eo[e] = (0.f + above[1][e]) + here[1][e];
      oe[e] = (0.f + here[0][e]) + here[1][e];
      oo[e] = 0.f + here[1][e];
    }
    const int y0 = 2 * br - p.pad_rows;
    const bool y_ok[2] = {
        static_cast<unsigned>(y0) < static_cast<unsigned>(p.in_rows),
        static_cast<unsigned>(y0 + 1) < static_cast<unsigned>(p.in_rows)};
    const unsigned base =
        static_cast<unsigned>(((n * p.in_rows + y0) * p.in_cols + x0) * C + ch) *
        kEsz;
    BufVec4<T>::store(dx_rsrc, (y_ok[0] && x_ok[0]) ? base : kOobOffset,
                          ee);
    BufVec4<T>::store(
        dx_rsrc, (y_ok[0] && x_ok[1]) ? base + col_bytes : kOobOffset, eo);
    BufVec4<T>::store(
        dx_rsrc, (y_ok[1] && x_ok[0]) ? base + row_bytes : kOobOffset, oe);
    BufVec4<T>::store(
        dx_rsrc,
        (y_ok[1] && x_ok[1]) ? base + row_bytes + col_bytes : kOobOffset, oo);
  }
}

template <typename T, typename Op>
int launch_forward_op(const T* input, T* output,
                      const snn_hip_pooling_params& p, hipStream_t stream) {
  constexpr int kBlock = 256;
  const size_t n_out =
      static_cast<size_t>(p.batch) * p.out_rows * p.out_cols * p.channels;
  const size_t in_bytes = static_cast<size_t>(p.batch) * p.in_rows *
                          p.in_cols * p.channels * sizeof(T);
  const bool is3x3 = p.window_rows == 3 && p.window_cols == 3 &&
                     p.stride_rows == p.stride_cols &&
                     (p.stride_rows == 1 || p.stride_rows == 2);
  // every window must overlap the image (the strip kernel redirects outside
  // taps to the nearest inside tap of the same window)
  const bool overlaps =
      p.pad_rows < 3 && p.pad_cols < 3 &&
      (p.out_rows - 1) * p.stride_rows - p.pad_rows < p.in_rows &&
      (p.out_cols - 1) * p.stride_cols - p.pad_cols < p.in_cols;
  // fp32, stride 2, 32 / 64 / 128 channels and enough waves to cover the GPU:
  // the tall-strip kernel
  bool tall = false;
  if constexpr (std::is_same<T, float>::value) {
    const int cv = p.channels / 4;
    constexpr int kTallRows = 7;
    const int pxw = cv > 0 ? 64 / cv : 0;
    if (p.channels % 4 == 0 && is3x3 && p.stride_rows == 2 &&
        (cv == 8 || cv == 16 || cv == 32) && p.out_rows >= kTallRows &&
        in_bytes < 0x7FFFFFF0u && n_out * sizeof(T) < 0x7FFFFFF0u &&
        SNN_TUNING_ENV("SNN_HIP_POOL_TALL_OFF") == nullptr) {
      const int n_wcols = ceil_div(p.out_cols, pxw);
      const int n_strips = ceil_div(p.out_rows, kTallRows);
      const size_t waves = static_cast<size_t>(p.batch) * n_strips * n_wcols;
      if (waves >= 768 && waves < 0x3FFFFFFFu &&
          static_cast<size_t>(n_wcols) * pxw * 4 <=
              static_cast<size_t>(p.out_cols) * 5) {
        const unsigned n_waves = static_cast<unsigned>(waves);
        const dim3 grid(ceil_div(n_waves, 4u));
#define SNN_POOL_TALL(CV)                                                      \
  hipLaunchKernelGGL((pool_forward_3x3_s2_tall_kernel<Op, kTallRows, CV>),    \
                     grid, dim3(kBlock), 0, stream, input, output, p,          \
                     n_strips, n_wcols, n_waves)
        if (cv == 8) SNN_POOL_TALL(8);
        else if (cv == 16) SNN_POOL_TALL(16);
        else SNN_POOL_TALL(32);
#undef SNN_POOL_TALL
        tall = true;
      }
    }
  }
  if (tall) {
    // launched above
  } else if (p.channels % 4 == 0 && is3x3 && overlaps &&
             in_bytes < 0x7FFFFFF0u && n_out * sizeof(T) < 0x7FFFFFF0u) {
    const size_t per_row =
        static_cast<size_t>(p.batch) * p.out_cols * (p.channels / 4);
    // Two output rows per lane: measured on MI355X with the XCD-contiguous
    // order above, the 112x112x64 stride-2 max pool runs in 24.4 us with one
    // or two rows per lane against 26.0 us with four (the rows that strips
    // share come from the XCD's L2 either way, and shorter strips leave more
    // lanes to keep loads in flight).
    int th = 2;
    while (th > 1 && per_row * ceil_div(p.out_rows, th) < 150000) th /= 2;
    // Developer override for tuning runs: SNN_HIP_POOL_TH=<1|2|4>.
    static const char* tune = SNN_TUNING_ENV("SNN_HIP_POOL_TH");
    if (tune != nullptr && tune[0] != 0) th = atoi(tune);
    th = th >= 4 ? 4 : th >= 2 ? 2 : 1;
    const int n_strips = ceil_div(p.out_rows, th);
    const unsigned n_items = static_cast<unsigned>(per_row * n_strips);
    const dim3 grid(ceil_div(n_items, static_cast<unsigned>(kBlock)));
#define SNN_POOL_STRIP(STRIDE, TH)                                             \
  hipLaunchKernelGGL((pool_forward_3x3_strip_kernel<T, Op, STRIDE, TH>), grid, \
                     dim3(kBlock), 0, stream, input, output, p, n_strips,      \
                     n_items)
    if (p.stride_rows == 1) {
      if (th == 4) SNN_POOL_STRIP(1, 4);
      else if (th == 2) SNN_POOL_STRIP(1, 2);
      else SNN_POOL_STRIP(1, 1);
    } else {
      if (th == 4) SNN_POOL_STRIP(2, 4);
      else if (th == 2) SNN_POOL_STRIP(2, 2);
      else SNN_POOL_STRIP(2, 1);
    }
#undef SNN_POOL_STRIP
  } else if (p.channels % 4 == 0 && p.window_rows * p.window_cols >= 16 &&
             n_out / 4 < 200000) {
    // few, large windows: split the window taps over the lanes
    const int n_groups = ceil_div(p.channels, 64);
    const unsigned blocks = static_cast<unsigned>(
        static_cast<size_t>(p.batch) * p.out_rows * p.out_cols * n_groups);
    hipLaunchKernelGGL((pool_forward_tapsplit_kernel<T, Op>), dim3(blocks),
                       dim3(kBlock), 0, stream, input, output, p, n_groups);
  } else if (p.channels % 4 == 0) {
    const size_t n_vec = n_out / 4;
    hipLaunchKernelGGL((pool_forward_kernel<T, Op, 4>),
                       dim3(static_cast<unsigned>(ceil_div(n_vec, size_t{kBlock}))),
                       dim3(kBlock), 0, stream, input, output, p, n_vec);
  } else {
    hipLaunchKernelGGL((pool_forward_kernel<T, Op, 1>),
                       dim3(static_cast<unsigned>(ceil_div(n_out, size_t{kBlock}))),
                       dim3(kBlock), 0, stream, input, output, p, n_out);
  }
  SNN_HIP_CHECK_LAUNCH();
  return SNN_HIP_OK;
}

// Max gradient for small square windows (WIN x WIN, stride STRIDE), four
// channels per lane.  The per-element kernel above re-scans a window for
// every input element that ties with its maximum; here a work-group owns a
// 16 x 16 tile of input pixels and up to 64 channels:
//   1. every window that touches the tile is scanned once (row-major, clipped
//      to the image) for the first element equal to the forward output -- the
//      reference's tie rule (src/pooling/kernels.h:197-239) -- and the
//      position WIN * r + c (255: none) of each channel goes to LDS;
//   2. every input element of the tile looks up the windows that cover it and
//      takes dY of those whose recorded position is its own.
// Windows on the tile border are scanned by both neighbouring tiles; nothing
// is accumulated across work-groups, so no atomics and no zero fill.
constexpr int kGradTile = 16;
template <int WIN, int STRIDE>
__global__ void __launch_bounds__(256)
    pool_max_grad_tile_kernel(const float* __restrict__ in,
                              const float* __restrict__ out,
                              const float* __restrict__ dy,
                              float* __restrict__ dx, snn_hip_pooling_params p,
                              bool nan_mode, int tiles_x, int tiles_y,
                              int cv_per_group) {
  // windows per dimension that can touch 16 consecutive input rows / columns
  constexpr int NW = (kGradTile + WIN - 2) / STRIDE + 2;
  constexpr int kMaxCv = 16;
  __shared__ unsigned int first_pos[NW * NW * kMaxCv];  // 4 channel bytes each

  const int C = p.channels;
  int t = blockIdx.x;
  const int tx = t % tiles_x;
  t /= tiles_x;
  const int ty = t % tiles_y;
  const int n = t / tiles_y;
  const int cv0 = blockIdx.y * cv_per_group;
  const int cvl = threadIdx.x % cv_per_group;
  const int lane_w = threadIdx.x / cv_per_group;
  const int n_lanes_w = 256 / cv_per_group;
  const int ch = (cv0 + cvl) * 4;
  const bool ch_ok = ch < C;

  const int iy0 = ty * kGradTile, ix0 = tx * kGradTile;
  // first window (per dimension) whose unclipped extent reaches the tile
  auto first_window = [](int i0, int pad) {
    const int v = i0 + pad - WIN + 1;  // smallest o with o*STRIDE - pad + WIN - 1 >= i0
    return v <= 0 ? 0 : (v + STRIDE - 1) / STRIDE;
  };
  const int oy0 = first_window(iy0, p.pad_rows);
  const int ox0 = first_window(ix0, p.pad_cols);
  const size_t in_base =
      static_cast<size_t>(n) * p.in_rows * p.in_cols * C + ch;
  const size_t out_base =
      static_cast<size_t>(n) * p.out_rows * p.out_cols * C + ch;

  for (int w = lane_w; w < NW * NW; w += n_lanes_w) {
    const int oy = oy0 + w / NW, ox = ox0 + w % NW;
    unsigned int packed = 0xFFFFFFFFu;
    if (ch_ok && oy < p.out_rows && ox < p.out_cols) {
      float target[4];
      GradVec<4>::load(
          out + out_base + (static_cast<size_t>(oy) * p.out_cols + ox) * C,
          target);
      unsigned int pos[4] = {255u, 255u, 255u, 255u};
      const int r_in = oy * STRIDE - p.pad_rows;
      const int c_in = ox * STRIDE - p.pad_cols;
#pragma unroll
      for (int r = 0; r < WIN; ++r) {
#pragma unroll
        for (int c = 0; c < WIN; ++c) {
          const int iy = r_in + r, ix = c_in + c;
          if (static_cast<unsigned>(iy) < static_cast<unsigned>(p.in_rows) &&
              static_cast<unsigned>(ix) < static_cast<unsigned>(p.in_cols)) {
            float v[4];
            GradVec<4>::load(
                in + in_base + (static_cast<size_t>(iy) * p.in_cols + ix) * C,
                v);
#pragma unroll
            for (int i = 0; i < 4; ++i)
              if (pos[i] == 255u && pool_equal(v[i], target[i], nan_mode))
                pos[i] = static_cast<unsigned>(r * WIN + c);
          }
        }
      }
      packed = pos[0] | (pos[1] << 8) | (pos[2] << 16) | (pos[3] << 24);
    }
    first_pos[w * kMaxCv + cvl] = packed;
  }
  __syncthreads();

  if (!ch_ok) return;
  for (int pix = lane_w; pix < kGradTile * kGradTile; pix += n_lanes_w) {
    const int iy = iy0 + pix / kGradTile, ix = ix0 + pix % kGradTile;
    if (iy >= p.in_rows || ix >= p.in_cols) continue;
    float grad[4] = {0.f, 0.f, 0.f, 0.f};
    // windows whose unclipped extent contains (iy, ix)
    const int py = iy + p.pad_rows, px = ix + p.pad_cols;
    const int oy_begin = py < WIN ? 0 : (py - WIN) / STRIDE + 1;
    const int oy_end = min(py / STRIDE + 1, p.out_rows);
    const int ox_begin = px < WIN ? 0 : (px - WIN) / STRIDE + 1;
    const int ox_end = min(px / STRIDE + 1, p.out_cols);
    for (int oy = oy_begin; oy < oy_end; ++oy) {
      for (int ox = ox_begin; ox < ox_end; ++ox) {
        const unsigned int mine = static_cast<unsigned>(
            (py - oy * STRIDE) * WIN + (px - ox * STRIDE));
        const unsigned int packed =
            first_pos[((oy - oy0) * NW + (ox - ox0)) * kMaxCv + cvl];
        bool hit[4];
        bool any = false;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          hit[i] = ((packed >> (8 * i)) & 255u) == mine;
          any |= hit[i];
        }
        if (!any) continue;
        float g[4];
        GradVec<4>::load(
            dy + out_base + (static_cast<size_t>(oy) * p.out_cols + ox) * C, g);
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (hit[i]) grad[i] += g[i];
      }
    }
    GradVec<4>::store(
        dx + in_base + (static_cast<size_t>(iy) * p.in_cols + ix) * C, grad);
  }
}

// Max gradient, 3x3 windows, stride 2, four channels per lane, without LDS.
// In padded coordinates t = y + pad window o covers t = 2 * o .. 2 * o + 2,
// so the 2 x 2 dX pixels of block (br, bc) (t rows 2 * br, 2 * br + 1, columns
// alike) are covered by windows (br - 1 .. br) x (bc - 1 .. bc) only.  A lane
// walks TH consecutive block rows of one block column: per block row it loads
// two input rows of five columns (the third row of the two new windows is the
// first row of the next block row and is carried in registers), finds for the
// windows (br, bc - 1) and (br, bc) the first element equal to the forward
// output in row-major order -- the reference's tie rule
// (src/pooling/kernels.h:197-239) -- and carries those two positions and dY
// values down as the "windows above" of the next block row.  Each dX pixel
// adds its windows in output-row, output-column order.
template <int TH, bool NAN_MODE, typename T = float>
__global__ void __launch_bounds__(256)
    pool_max_grad_3x3_s2_kernel(const T* __restrict__ in,
                                const T* __restrict__ out,
                                const T* __restrict__ dy,
                                T* __restrict__ dx, snn_hip_pooling_params p,
                                int n_bcols, int n_strips, unsigned n_items) {
  constexpr bool nan_mode = NAN_MODE;
  const unsigned idx = blockIdx.x * 256u + threadIdx.x;
  if (idx >= n_items) return;
  const int C = p.channels;
  const unsigned cv = static_cast<unsigned>(C) / 4u;
  const int ch = static_cast<int>(idx % cv) * 4;
  unsigned t = idx / cv;
  const int bc = static_cast<int>(t % static_cast<unsigned>(n_bcols)) +
                 p.pad_cols / 2;
  t /= static_cast<unsigned>(n_bcols);
  const int br0 = static_cast<int>(t % static_cast<unsigned>(n_strips)) * TH +
                  p.pad_rows / 2;
  const int n = static_cast<int>(t / static_cast<unsigned>(n_strips));
  constexpr unsigned kEsz = sizeof(T);
  const size_t in_elems =
      static_cast<size_t>(p.batch) * p.in_rows * p.in_cols * C;
  const size_t out_elems =
      static_cast<size_t>(p.batch) * p.out_rows * p.out_cols * C;
  const __amdgpu_buffer_rsrc_t in_rsrc = make_rsrc(in, in_elems * kEsz);
  const __amdgpu_buffer_rsrc_t out_rsrc = make_rsrc(out, out_elems * kEsz);
  const __amdgpu_buffer_rsrc_t dy_rsrc = make_rsrc(dy, out_elems * kEsz);
  const __amdgpu_buffer_rsrc_t dx_rsrc = make_rsrc(dx, in_elems * kEsz);

  // input columns 2 * bc - 2 .. 2 * bc + 2 (padded), image column x0 + j
  const int x0 = 2 * bc - 2 - p.pad_cols;
  bool x_ok[5];
#pragma unroll
  for (int j = 0; j < 5; ++j)
    x_ok[j] = static_cast<unsigned>(x0 + j) < static_cast<unsigned>(p.in_cols);
  // windows bc - 1 and bc
  const bool w_ok[2] = {bc >= 1 && bc - 1 < p.out_cols, bc < p.out_cols};
  const unsigned in_row_bytes = static_cast<unsigned>(p.in_cols * C) * kEsz;
  const unsigned in_image = static_cast<unsigned>(n * p.in_rows) * in_row_bytes;
  const unsigned in_col0 = static_cast<unsigned>(x0 * C + ch) * kEsz;
  // (Offsets outside the image are made out of range with mask arithmetic,
  // not with a conditional: the compiler turns a per-lane condition around
  // these loads into two branches that load into the same registers and waits
  // for every load in flight between them.)
  unsigned x_bad[5];
#pragma unroll
  for (int j = 0; j < 5; ++j) x_bad[j] = 0u - static_cast<unsigned>(!x_ok[j]);
  auto load_in_row = [&](int y, float (&v)[5][4]) {
    const unsigned y_bad = 0u - static_cast<unsigned>(
                                    static_cast<unsigned>(y) >=
                                    static_cast<unsigned>(p.in_rows));
    const unsigned base =
        in_image + static_cast<unsigned>(y) * in_row_bytes + in_col0;
#pragma unroll
    for (int j = 0; j < 5; ++j) {
      const unsigned bad = y_bad | x_bad[j];
      BufVec4<T>::load(
          in_rsrc,
          ((base + static_cast<unsigned>(j * C) * kEsz) & ~bad) |
              (kOobOffset & bad),
          v[j]);
    }
  };
  const unsigned w_bad[2] = {0u - static_cast<unsigned>(!w_ok[0]),
                             0u - static_cast<unsigned>(!w_ok[1])};
  auto load_out_pair = [&](__amdgpu_buffer_rsrc_t rsrc, int oy,
                           float (&v)[2][4]) {
    const unsigned oy_bad = 0u - static_cast<unsigned>(
                                     static_cast<unsigned>(oy) >=
                                     static_cast<unsigned>(p.out_rows));
    const unsigned base = static_cast<unsigned>(
        ((n * p.out_rows + oy) * p.out_cols + bc - 1) * C + ch) * kEsz;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const unsigned bad = oy_bad | w_bad[j];
      BufVec4<T>::load(
          rsrc,
          ((base + static_cast<unsigned>(j * C) * kEsz) & ~bad) |
              (kOobOffset & bad),
          v[j]);
    }
  };

  // windows of the block row above: first-maximum position (9: none) and dY
  int up_pos[2][4];
  float up_g[2][4];
  float rows[3][5][4];  // rows[0] is carried from the block row above
  {
    // block row br0 - 1, needed only for its windows: scan it in full
    const int y = 2 * (br0 - 1) - p.pad_rows;
    float target[2][4];
    load_out_pair(out_rsrc, br0 - 1, target);
    load_out_pair(dy_rsrc, br0 - 1, up_g);
    load_in_row(y, rows[0]);
    load_in_row(y + 1, rows[1]);
    load_in_row(y + 2, rows[2]);
    const bool win_row_ok = static_cast<unsigned>(br0 - 1) <
                            static_cast<unsigned>(p.out_rows);
    const bool interior =
        y >= 0 && y + 2 < p.in_rows && x_ok[0] && x_ok[1] && x_ok[2] &&
        x_ok[3] && x_ok[4] && win_row_ok && w_ok[0] && w_ok[1];
    if (__builtin_amdgcn_ballot_w64(!interior) == 0) {
#pragma unroll
      for (int w = 0; w < 2; ++w)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          int pos = 9;
#pragma unroll
          for (int k = 8; k >= 0; --k)
            if (pool_equal(rows[k / 3][2 * w + k % 3][e], target[w][e],
                           nan_mode))
              pos = k;
          up_pos[w][e] = pos;
        }
    } else {
#pragma unroll
      for (int w = 0; w < 2; ++w)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          int pos = 9;
#pragma unroll
          for (int k = 8; k >= 0; --k) {
            const int r = k / 3, c = k % 3;
            const bool y_ok = static_cast<unsigned>(y + r) <
                              static_cast<unsigned>(p.in_rows);
            if (y_ok && x_ok[2 * w + c] &&
                pool_equal(rows[r][2 * w + c][e], target[w][e], nan_mode))
              pos = k;
          }
          up_pos[w][e] = (win_row_ok && w_ok[w]) ? pos : 9;
        }
    }
#pragma unroll
    for (int j = 0; j < 5; ++j)
#pragma unroll
      for (int e = 0; e < 4; ++e) rows[0][j][e] = rows[2][j][e];
  }

  // The four dX pixels of a block row are stored after the next block row's
  // loads have been issued: vector-memory operations retire in order, so
  // stores issued before those loads would have to be acknowledged before
  // the loads' data could be used.
  float ee[4], eo[4], oe[4], oo[4];
  unsigned st_off[4];
  auto store_block_row = [&]() {
    BufVec4<T>::store(dx_rsrc, st_off[0], ee);
    BufVec4<T>::store(dx_rsrc, st_off[1], eo);
    BufVec4<T>::store(dx_rsrc, st_off[2], oe);
    BufVec4<T>::store(dx_rsrc, st_off[3], oo);
  };
  // (short strips unrolled in full; nothing in the body is indexed by i, so the
  // 14-row strip runs as a loop of two block rows a turn -- one a turn
  // measured 62 us, two or seven 57)
#pragma unroll TH <= 4 ? TH : 2
  for (int i = 0; i < TH; ++i) {
    const int br = br0 + i;
    const int y = 2 * br - p.pad_rows;  // image row of padded row 2 * br
    float target[2][4], g[2][4];
    load_out_pair(out_rsrc, br, target);
    load_out_pair(dy_rsrc, br, g);
    load_in_row(y + 1, rows[1]);
    load_in_row(y + 2, rows[2]);
    __builtin_amdgcn_sched_barrier(0);
    if (i > 0) store_block_row();
    __builtin_amdgcn_sched_barrier(0);
    bool y_ok[3];
#pragma unroll
    for (int r = 0; r < 3; ++r)
      y_ok[r] = static_cast<unsigned>(y + r) < static_cast<unsigned>(p.in_rows);
    const bool win_row_ok =
        static_cast<unsigned>(br) < static_cast<unsigned>(p.out_rows);
    int pos[2][4];
    // Away from the image border every element of both windows exists for
    // every lane of the wave: the search then is a compare and a select per
    // element, with none of the per-element validity masks (scalar mask
    // arithmetic that outnumbered the vector instructions of this kernel).
    const bool interior = y_ok[0] && y_ok[1] && y_ok[2] && x_ok[0] &&
                          x_ok[1] && x_ok[2] && x_ok[3] && x_ok[4] &&
                          win_row_ok && w_ok[0] && w_ok[1];
    if (__builtin_amdgcn_ballot_w64(!interior) == 0) {
#pragma unroll
      for (int w = 0; w < 2; ++w)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          int first = 9;
#pragma unroll
          for (int k = 8; k >= 0; --k)
            if (pool_equal(rows[k / 3][2 * w + k % 3][e], target[w][e],
                           nan_mode))
              first = k;
          pos[w][e] = first;
        }
    } else {
#pragma unroll
      for (int w = 0; w < 2; ++w)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          int first = 9;
#pragma unroll
          for (int k = 8; k >= 0; --k) {
            const int r = k / 3, c = k % 3;
            if (y_ok[r] && x_ok[2 * w + c] &&
                pool_equal(rows[r][2 * w + c][e], target[w][e], nan_mode))
              first = k;
          }
          pos[w][e] = (win_row_ok && w_ok[w]) ? first : 9;
        }
    }
    // the four dX pixels; windows in (output row, output column) order
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      float v = 0.f;
      if (up_pos[0][e] == 8) v += up_g[0][e];
      if (up_pos[1][e] == 6) v += up_g[1][e];
      if (pos[0][e] == 2) v += g[0][e];
      if (pos[1][e] == 0) v += g[1][e];
      ee[e] = v;
      v = 0.f;
      if (up_pos[1][e] == 7) v += up_g[1][e];
      if (pos[1][e] == 1) v += g[1][e];
      eo[e] = v;
      v = 0.f;
      if (pos[0][e] == 5) v += g[0][e];
      if (pos[1][e] == 3) v += g[1][e];
      oe[e] = v;
      oo[e] = pos[1][e] == 4 ? 0.f + g[1][e] : 0.f;
    }
    const unsigned base = in_image + static_cast<unsigned>(y) * in_row_bytes +
                          in_col0 + static_cast<unsigned>(2 * C) * kEsz;
    const unsigned col_bytes = static_cast<unsigned>(C) * kEsz;
    st_off[0] = (y_ok[0] && x_ok[2]) ? base : kOobOffset;
    st_off[1] = (y_ok[0] && x_ok[3]) ? base + col_bytes : kOobOffset;
    st_off[2] = (y_ok[1] && x_ok[2]) ? base + in_row_bytes : kOobOffset;
    st_off[3] =
        (y_ok[1] && x_ok[3]) ? base + in_row_bytes + col_bytes : kOobOffset;
#pragma unroll
    for (int w = 0; w < 2; ++w)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        up_pos[w][e] = pos[w][e];
        up_g[w][e] = g[w][e];
      }
#pragma unroll
    for (int j = 0; j < 5; ++j)
#pragma unroll
      for (int e = 0; e < 4; ++e) rows[0][j][e] = rows[2][j][e];
  }
  store_block_row();
}

template <int WIN, int STRIDE>
void launch_max_grad_tile(const float* in, const float* out, const float* dy,
                          float* dx, const snn_hip_pooling_params& p,
                          bool nan_mode, hipStream_t stream) {
  const int cv = p.channels / 4;
  int cv_per_group = 16;
  while (cv_per_group > 1 && cv_per_group / 2 >= cv) cv_per_group /= 2;
  const int tiles_x = ceil_div(p.in_cols, kGradTile);
  const int tiles_y = ceil_div(p.in_rows, kGradTile);
  // A work-group's lanes walk the tile's windows and pixels in turns of 256 /
  // cv_per_group: with few tiles, fewer channels per work-group give more
  // work-groups and shorter turns (56x56x64 at batch 16: 256 work-groups of
  // 20 + 16 turns took 143 us, 1024 of 5 + 4 turns 54 us; going on to 4096
  // work-groups or 32 contiguous bytes per pixel measured slower).
  while (cv_per_group > 4 &&
         static_cast<long>(p.batch) * tiles_y * tiles_x *
                 ceil_div(cv, cv_per_group) < 2048)
    cv_per_group /= 2;
  const dim3 grid(static_cast<unsigned>(p.batch * tiles_y * tiles_x),
                  static_cast<unsigned>(ceil_div(cv, cv_per_group)));
  hipLaunchKernelGGL((pool_max_grad_tile_kernel<WIN, STRIDE>), grid, dim3(256),
                     0, stream, in, out, dy, dx, p, nan_mode, tiles_x, tiles_y,
                     cv_per_group);
}

// The 3x3 stride-2 max gradient without LDS (pool_max_grad_3x3_s2_kernel),
// fp32 or binary16 tensors.
template <typename T>
void launch_max_grad_3x3_s2(const T* input_data, const T* output_data,
                            const T* input_backprop, T* output_backprop,
                            const snn_hip_pooling_params& p, bool nan_mode,
                            hipStream_t stream) {
  constexpr int kBlock = 256;
  // block rows / columns: padded coordinates pad .. in + pad - 1, halved
  const int n_brows = (p.in_rows + p.pad_rows - 1) / 2 - p.pad_rows / 2 + 1;
  const int n_bcols = (p.in_cols + p.pad_cols - 1) / 2 - p.pad_cols / 2 + 1;
  const size_t per_row =
      static_cast<size_t>(p.batch) * n_bcols * (p.channels / 4);
  // Block rows per lane: a strip re-reads the three input rows and the
  // output / dY row of the block row above it, so the longest strip that
  // still leaves about six waves per CU (112x112x64 at batch 32: 14 block
  // rows, 1.1 x the input read instead of 1.4 x, 60 -> 56 us; 28 leave 3.5
  // waves per CU: 76 us).
  int th = per_row * ceil_div(n_brows, 14) >= 100000
               ? 14
               : per_row * ceil_div(n_brows, 4) >= 150000 ? 4 : 2;
  if (const char* tune = SNN_TUNING_ENV("SNN_HIP_POOL_GRAD_TH")) {
    const int v = std::atoi(tune);
    if (v == 2 || v == 4 || v == 14) th = v;
  }
  const int n_strips = ceil_div(n_brows, th);
  const unsigned n_items = static_cast<unsigned>(per_row * n_strips);
  const dim3 grid(ceil_div(n_items, static_cast<unsigned>(kBlock)));
  auto launch = [&](auto kernel) {
    hipLaunchKernelGGL(kernel, grid, dim3(kBlock), 0, stream, input_data,
                       output_data, input_backprop, output_backprop, p,
                       n_bcols, n_strips, n_items);
  };
  if (th == 14) {
    if (nan_mode)
      launch(pool_max_grad_3x3_s2_kernel<14, true, T>);
    else
      launch(pool_max_grad_3x3_s2_kernel<14, false, T>);
  } else if (th == 4) {
    if (nan_mode)
      launch(pool_max_grad_3x3_s2_kernel<4, true, T>);
    else
      launch(pool_max_grad_3x3_s2_kernel<4, false, T>);
  } else {
    if (nan_mode)
      launch(pool_max_grad_3x3_s2_kernel<2, true, T>);
    else
      launch(pool_max_grad_3x3_s2_kernel<2, false, T>);
  }
}

// The 3x3 stride-2 average gradient (pool_avg_grad_3x3_s2_kernel), fp32 or
// binary16 tensors.
template <typename T>
void launch_avg_grad_3x3_s2(const T* input_backprop, T* output_backprop,
                            const snn_hip_pooling_params& p,
                            hipStream_t stream) {
  constexpr int kBlock = 256;
  // block rows / columns: padded coordinates pad .. in + pad - 1, halved
  const int n_brows = (p.in_rows + p.pad_rows - 1) / 2 - p.pad_rows / 2 + 1;
  const int n_bcols = (p.in_cols + p.pad_cols - 1) / 2 - p.pad_cols / 2 + 1;
  const size_t per_row =
      static_cast<size_t>(p.batch) * n_bcols * (p.channels / 4);
  const int th = per_row * ceil_div(n_brows, 4) >= 150000 ? 4 : 2;
  const int n_strips = ceil_div(n_brows, th);
  const unsigned n_items = static_cast<unsigned>(per_row * n_strips);
  const dim3 grid(ceil_div(n_items, static_cast<unsigned>(kBlock)));
  if (th == 4)
    hipLaunchKernelGGL((pool_avg_grad_3x3_s2_kernel<4, T>), grid, dim3(kBlock), 0,
                       stream, input_backprop, output_backprop, p, n_bcols,
                       n_strips, n_items);
  else
    hipLaunchKernelGGL((pool_avg_grad_3x3_s2_kernel<2, T>), grid, dim3(kBlock), 0,
                       stream, input_backprop, output_backprop, p, n_bcols,
                       n_strips, n_items);
}

}  // namespace

template <typename T>
int launch_pooling_forward(const T* input, T* output,
                           const snn_hip_pooling_params& p, int op,
                           hipStream_t stream) {
  KernelTimer timer(stream);
  switch (op) {
    case SNN_HIP_POOL_MAX:
      return launch_forward_op<T, MaxOp>(input, output, p, stream);
    case SNN_HIP_POOL_MAX_WITH_NAN:
      return launch_forward_op<T, MaxNanOp>(input, output, p, stream);
    case SNN_HIP_POOL_AVERAGE:
      return launch_forward_op<T, AvgOp>(input, output, p, stream);
    default:
      return SNN_HIP_INVALID_PARAMETER;
  }
}

template int launch_pooling_forward<float>(const float*, float*,
                                           const snn_hip_pooling_params&, int,
                                           hipStream_t);
template int launch_pooling_forward<_Float16>(const _Float16*, _Float16*,
                                              const snn_hip_pooling_params&,
                                              int, hipStream_t);

static inline bool grad_aligned16(const void* ptr) {
  return (reinterpret_cast<uintptr_t>(ptr) & 15u) == 0;
}

int launch_pooling_max_grad(const float* input_data, const float* output_data,
                            const float* input_backprop,
                            float* output_backprop,
                            const snn_hip_pooling_params& p, int op,
                            hipStream_t stream) {
  KernelTimer timer(stream);
  constexpr int kBlock = 256;
  const size_t n_in =
      static_cast<size_t>(p.batch) * p.in_rows * p.in_cols * p.channels;
  const bool nan_mode = op == SNN_HIP_POOL_MAX_WITH_NAN;
  const bool vec4 = p.channels % 4 == 0 && grad_aligned16(input_data) &&
                    grad_aligned16(output_data) &&
                    grad_aligned16(input_backprop) &&
                    grad_aligned16(output_backprop);
  const bool square = p.window_rows == p.window_cols &&
                      p.stride_rows == p.stride_cols &&
                      static_cast<size_t>(p.batch) *
                              ceil_div(p.in_rows, kGradTile) *
                              ceil_div(p.in_cols, kGradTile) < 0x7FFFFFFFu &&
                      ceil_div(p.channels / 4, 16) <= 65535;
  const size_t n_out =
      static_cast<size_t>(p.batch) * p.out_rows * p.out_cols * p.channels;
  static const bool use_tiles = SNN_TUNING_ENV("SNN_HIP_POOL_GRAD_TILES") != nullptr;
  if (vec4 && square && p.window_rows == 3 && p.stride_rows == 2 &&
      !use_tiles && n_in * 4 < 0x7FFFFFF0u && n_out * 4 < 0x7FFFFFF0u) {
    launch_max_grad_3x3_s2<float>(input_data, output_data, input_backprop,
                                  output_backprop, p, nan_mode, stream);
  } else if (vec4 && square && p.window_rows == 3 && p.stride_rows == 2) {
    launch_max_grad_tile<3, 2>(input_data, output_data, input_backprop,
                               output_backprop, p, nan_mode, stream);
  } else if (vec4 && square && p.window_rows == 3 && p.stride_rows == 1) {
    launch_max_grad_tile<3, 1>(input_data, output_data, input_backprop,
                               output_backprop, p, nan_mode, stream);
  } else if (vec4 && square && p.window_rows == 2 && p.stride_rows == 2) {
    launch_max_grad_tile<2, 2>(input_data, output_data, input_backprop,
                               output_backprop, p, nan_mode, stream);
  } else if (vec4) {
    const size_t n_vec = n_in / 4;
    hipLaunchKernelGGL(pool_max_grad_kernel<4>,
                       dim3(static_cast<unsigned>(ceil_div(n_vec, size_t{kBlock}))),
                       dim3(kBlock), 0, stream, input_data, output_data,
                       input_backprop, output_backprop, p, nan_mode, n_vec);
  } else {
    hipLaunchKernelGGL(pool_max_grad_kernel<1>,
                       dim3(static_cast<unsigned>(ceil_div(n_in, size_t{kBlock}))),
                       dim3(kBlock), 0, stream, input_data, output_data,
                       input_backprop, output_backprop, p, nan_mode, n_in);
  }
  SNN_HIP_CHECK_LAUNCH();
  return SNN_HIP_OK;
}

int launch_pooling_avg_grad(const float* input_backprop,
                            float* output_backprop,
                            const snn_hip_pooling_params& p,
                            hipStream_t stream) {
  KernelTimer timer(stream);
  constexpr int kBlock = 256;
  const size_t n_in =
      static_cast<size_t>(p.batch) * p.in_rows * p.in_cols * p.channels;
  const size_t n_out =
      static_cast<size_t>(p.batch) * p.out_rows * p.out_cols * p.channels;
  static const bool no_s2 = SNN_TUNING_ENV("SNN_HIP_POOL_AVG_GRAD_GENERIC") != nullptr;
  if (p.channels % 4 == 0 && grad_aligned16(input_backprop) &&
      grad_aligned16(output_backprop) && p.window_rows == 3 &&
      p.window_cols == 3 && p.stride_rows == 2 && p.stride_cols == 2 &&
      n_in * 4 < 0x7FFFFFF0u && n_out * 4 < 0x7FFFFFF0u && !no_s2) {
    launch_avg_grad_3x3_s2<float>(input_backprop, output_backprop, p, stream);
  } else if (p.channels % 4 == 0 && grad_aligned16(input_backprop) &&
             grad_aligned16(output_backprop)) {
    const size_t n_vec = n_in / 4;
    // row strips when they still give every CU a few thousand lanes
    const size_t per_row =
        static_cast<size_t>(p.batch) * p.in_cols * (p.channels / 4);
    int th = 8;
    while (th > 1 && per_row * ceil_div(p.in_rows, th) < 150000) th /= 2;
    static const char* tune = SNN_TUNING_ENV("SNN_HIP_POOL_GRAD_TH");
    if (tune != nullptr && tune[0] != 0) th = atoi(tune);
    const int n_strips = ceil_div(p.in_rows, th >= 8 ? 8 : 4);
    const size_t n_items = per_row * n_strips;
    if (th >= 4 && n_items < 0x7FFFFFFFu) {
      const dim3 grid(static_cast<unsigned>(ceil_div(n_items, size_t{kBlock})));
      if (th >= 8)
        hipLaunchKernelGGL(pool_avg_grad_strip_kernel<8>, grid, dim3(kBlock), 0,
                           stream, input_backprop, output_backprop, p, n_strips,
                           static_cast<unsigned>(n_items));
      else
        hipLaunchKernelGGL(pool_avg_grad_strip_kernel<4>, grid, dim3(kBlock), 0,
                           stream, input_backprop, output_backprop, p, n_strips,
                           static_cast<unsigned>(n_items));
    } else {
      hipLaunchKernelGGL(
          pool_avg_grad_kernel<4>,
          dim3(static_cast<unsigned>(ceil_div(n_vec, size_t{kBlock}))),
          dim3(kBlock), 0, stream, input_backprop, output_backprop, p, n_vec);
    }
  } else {
    hipLaunchKernelGGL(pool_avg_grad_kernel<1>,
                       dim3(static_cast<unsigned>(ceil_div(n_in, size_t{kBlock}))),
                       dim3(kBlock), 0, stream, input_backprop,
                       output_backprop, p, n_in);
  }
  SNN_HIP_CHECK_LAUNCH();
  return SNN_HIP_OK;
}

// Half-precision gradients (fp32 arithmetic inside a lane): the
// one-lane-per-element kernels, four channels per lane when the channel count
// and the pointers allow 8-byte accesses.
static inline bool grad_aligned8(const void* ptr) {
  return (reinterpret_cast<uintptr_t>(ptr) & 7u) == 0;
}

int launch_pooling_max_grad_f16(const _Float16* input_data,
                                const _Float16* output_data,
                                const _Float16* input_backprop,
                                _Float16* output_backprop,
                                const snn_hip_pooling_params& p, int op,
                                hipStream_t stream) {
  KernelTimer timer(stream);
  constexpr int kBlock = 256;
  const size_t n_in =
      static_cast<size_t>(p.batch) * p.in_rows * p.in_cols * p.channels;
  const bool nan_mode = op == SNN_HIP_POOL_MAX_WITH_NAN;
  const size_t n_out =
      static_cast<size_t>(p.batch) * p.out_rows * p.out_cols * p.channels;
  if (p.channels % 4 == 0 && grad_aligned8(input_data) &&
      grad_aligned8(output_data) && grad_aligned8(input_backprop) &&
      grad_aligned8(output_backprop) && p.window_rows == 3 &&
      p.window_cols == 3 && p.stride_rows == 2 && p.stride_cols == 2 &&
      n_in * 2 < 0x7FFFFFF0u && n_out * 2 < 0x7FFFFFF0u) {
    // the fp32 kernel for this window, reading and writing binary16
    launch_max_grad_3x3_s2<_Float16>(input_data, output_data, input_backprop,
                                     output_backprop, p, nan_mode, stream);
  } else if (p.channels % 4 == 0 && grad_aligned8(input_data) &&
      grad_aligned8(output_data) && grad_aligned8(input_backprop) &&
      grad_aligned8(output_backprop)) {
    const size_t n_vec = n_in / 4;
    hipLaunchKernelGGL((pool_max_grad_kernel<4, _Float16>),
                       dim3(static_cast<unsigned>(ceil_div(n_vec, size_t{kBlock}))),
                       dim3(kBlock), 0, stream, input_data, output_data,
                       input_backprop, output_backprop, p, nan_mode, n_vec);
  } else {
    hipLaunchKernelGGL((pool_max_grad_kernel<1, _Float16>),
                       dim3(static_cast<unsigned>(ceil_div(n_in, size_t{kBlock}))),
                       dim3(kBlock), 0, stream, input_data, output_data,
                       input_backprop, output_backprop, p, nan_mode, n_in);
  }
  SNN_HIP_CHECK_LAUNCH();
  return SNN_HIP_OK;
}

int launch_pooling_avg_grad_f16(const _Float16* input_backprop,
                                _Float16* output_backprop,
                                const snn_hip_pooling_params& p,
                                hipStream_t stream) {
  KernelTimer timer(stream);
  constexpr int kBlock = 256;
  const size_t n_in =
      static_cast<size_t>(p.batch) * p.in_rows * p.in_cols * p.channels;
  const size_t n_out =
      static_cast<size_t>(p.batch) * p.out_rows * p.out_cols * p.channels;
  if (p.channels % 4 == 0 && grad_aligned8(input_backprop) &&
      grad_aligned8(output_backprop) && p.window_rows == 3 &&
      p.window_cols == 3 && p.stride_rows == 2 && p.stride_cols == 2 &&
      n_in * 2 < 0x7FFFFFF0u && n_out * 2 < 0x7FFFFFF0u) {
    // the fp32 kernel for this window, reading and writing binary16
    launch_avg_grad_3x3_s2<_Float16>(input_backprop, output_backprop, p,
                                     stream);
  } else if (p.channels % 4 == 0 && grad_aligned8(input_backprop) &&
      grad_aligned8(output_backprop)) {
    const size_t n_vec = n_in / 4;
    hipLaunchKernelGGL((pool_avg_grad_kernel<4, _Float16>),
                       dim3(static_cast<unsigned>(ceil_div(n_vec, size_t{kBlock}))),
                       dim3(kBlock), 0, stream, input_backprop,
                       output_backprop, p, n_vec);
  } else {
    hipLaunchKernelGGL((pool_avg_grad_kernel<1, _Float16>),
                       dim3(static_cast<unsigned>(ceil_div(n_in, size_t{kBlock}))),
                       dim3(kBlock), 0, stream, input_backprop,
                       output_backprop, p, n_in);
  }
  SNN_HIP_CHECK_LAUNCH();
  return SNN_HIP_OK;
}

}  // namespace snn
