// Depthwise convolution for gfx950: bandwidth-bound kernels, no MFMA.
// Stand-ins for portDNN's DepthwiseConv2D functors
// (src/depthwise_conv2d/kernels.h:40-366).
//
// Layout: input/output NHWC, filter [R][S][C][multiplier], output channel
// c*multiplier+j.
//
// Forward, multiplier 1, C % 4 == 0 (the MobileNet shapes): one lane owns a
// float4 (or 4 x f16) of channels, so the 64 lanes of a wave read one
// contiguous 1 KiB (512 B for f16) run of the NHWC row -- fully coalesced --
// and the window taps of neighbouring lanes/pixels are served from L1/L2.
// Everything else goes through the scalar kernel.
#include <cstdio>
#include <cstdlib>
#include <mutex>
#include <string>
#include <type_traits>

#include "gemm_tile.h"
#include "snn_kernels.h"

namespace snn {
namespace {

template <typename T>
struct Vec4;
template <>
struct Vec4<float> {
  using type = float4;
  __device__ static void load(const float* p, float (&v)[4]) {
    const float4 t = *reinterpret_cast<const float4*>(p);
    v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
  }
  __device__ static void store(float* p, const float (&v)[4]) {
    *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
  }
};
template <>
struct Vec4<_Float16> {
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

// Forward, multiplier == 1, four channels per lane.
template <typename T>
__global__ void __launch_bounds__(256)
    dw_forward_vec4_kernel(const T* __restrict__ in, const T* __restrict__ fil,
                           T* __restrict__ out, snn_hip_depthwise_params p,
                           size_t n_vec) {
  const size_t idx = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (idx >= n_vec) return;
  const int C = p.channels;
  const int cv = C / 4;
  const int c = static_cast<int>(idx % cv) * 4;
  size_t pix = idx / cv;
  const int ox = static_cast<int>(pix % p.out_cols);
  pix /= p.out_cols;
  const int oy = static_cast<int>(pix % p.out_rows);
  const int n = static_cast<int>(pix / p.out_rows);
  const T* in_n = in + static_cast<size_t>(n) * p.in_rows * p.in_cols * C + c;
  const T* fil_c = fil + c;
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  const int y0 = oy * p.stride_rows - p.pad_rows;
  const int x0 = ox * p.stride_cols - p.pad_cols;
  for (int r = 0; r < p.window_rows; ++r) {
    const int y = y0 + r;
    if (y < 0 || y >= p.in_rows) continue;
    for (int s = 0; s < p.window_cols; ++s) {
      const int x = x0 + s;
      if (x < 0 || x >= p.in_cols) continue;
      float iv[4], fv[4];
      Vec4<T>::load(in_n + (static_cast<size_t>(y) * p.in_cols + x) * C, iv);
      Vec4<T>::load(fil_c + static_cast<size_t>(r * p.window_cols + s) * C, fv);
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[i] = fmaf(iv[i], fv[i], acc[i]);
    }
  }
  Vec4<T>::store(out + idx * 4, acc);
}

// Forward 3x3, multiplier == 1, four channels per lane, TH consecutive output
// rows per lane.  Every input row of the strip is loaded once (three column
// taps) and added into each of the up to three output rows it belongs to, so
// the reuse between vertically adjacent windows happens in registers and each
// lane keeps (TH - 1) * STRIDE + 3 independent row loads in flight.  Per
// output the taps are still accumulated in filter-row, filter-column order.
// Raw buffer access: an out-of-range byte offset reads zeros / drops the store,
// which turns the padding border into plain, branch-free loads.
typedef unsigned int uint4v __attribute__((ext_vector_type(4)));
typedef unsigned int uint2v __attribute__((ext_vector_type(2)));
constexpr unsigned kOobOffset = 0x7FFFFFF0u;
// Cache policy bits of the input loads (0 = default; a build-time switch for
// experiments, e.g. -DSNN_MEM_LOAD_AUX=2 for streaming loads).
#ifndef SNN_MEM_LOAD_AUX
#define SNN_MEM_LOAD_AUX 0
#endif
// Output is written once and not re-read by the kernel: stream it (slc).
constexpr int kStoreAux = 2;

__device__ inline __amdgpu_buffer_rsrc_t make_rsrc(const void* p, size_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(
      const_cast<void*>(p), 0,
      static_cast<unsigned>(bytes > 0x7FFFFFF0u ? 0x7FFFFFF0u : bytes),
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
        0, kStoreAux);
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
                                          0, kStoreAux);
  }
};

// V channels per lane: 4 (16 bytes of fp32, 8 bytes of f16) or, for f16, 8
// (16 bytes).
template <typename T, int V>
struct BufVecN : BufVec4<T> {};
template <>
struct BufVecN<_Float16, 8> {
  typedef _Float16 half8 __attribute__((ext_vector_type(8)));
  __device__ static void load(__amdgpu_buffer_rsrc_t r, unsigned off,
                              float (&v)[8]) {
    const half8 t = __builtin_bit_cast(
        half8, __builtin_amdgcn_raw_buffer_load_b128(r, off, 0, SNN_MEM_LOAD_AUX));
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = static_cast<float>(t[i]);
  }
  __device__ static void store(__amdgpu_buffer_rsrc_t r, unsigned off,
                               const float (&v)[8]) {
    half8 t;
#pragma unroll
    for (int i = 0; i < 8; ++i) t[i] = static_cast<_Float16>(v[i]);
    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(uint4v, t), r,
                                           off, 0, kStoreAux);
  }
};

// Forward 3x3, multiplier == 1, four channels per lane, a TH x TW block of
// outputs per lane.  Every input row of the block is loaded once
// ((TW - 1) * STRIDE + 3 column taps) and added into each output row / column
// it belongs to, so the reuse between adjacent windows happens in registers.
// Per output the taps are still accumulated in filter-row, filter-column
// order.
// FLIP reads the filter taps in reverse order: with the output gradient as
// "input" and padding 2 - pad this is the stride-1 input gradient.
template <typename T, int STRIDE, int TH, int TW, bool FLIP = false, int V = 4>
__global__ void __launch_bounds__(256)
    dw_forward_3x3_strip_kernel(const T* __restrict__ in,
                                const T* __restrict__ fil, T* __restrict__ out,
                                snn_hip_depthwise_params p, int n_strips,
                                int n_col_blocks, unsigned n_items) {
  // Work-groups go round-robin to the 8 XCDs; remapping gives every XCD one
  // contiguous run of the index space, so vertically adjacent strips (which
  // share two input rows) meet in the same L2.
  const unsigned idx =
      gemm::xcd_remap(blockIdx.x, gridDim.x) * 256u + threadIdx.x;
  if (idx >= n_items) return;
  const int C = p.channels;
  const unsigned cv = static_cast<unsigned>(C) / V;
  const int c = static_cast<int>(idx % cv) * V;
  unsigned rest = idx / cv;
  const int ox0 =
      static_cast<int>(rest % static_cast<unsigned>(n_col_blocks)) * TW;
  rest /= static_cast<unsigned>(n_col_blocks);
  const int strip = static_cast<int>(rest % static_cast<unsigned>(n_strips));
  const int n = static_cast<int>(rest / static_cast<unsigned>(n_strips));
  const int oy0 = strip * TH;
  const size_t in_elems =
      static_cast<size_t>(p.batch) * p.in_rows * p.in_cols * C;
  const size_t out_elems =
      static_cast<size_t>(p.batch) * p.out_rows * p.out_cols * C;
  const __amdgpu_buffer_rsrc_t in_rsrc = make_rsrc(in, in_elems * sizeof(T));
  const __amdgpu_buffer_rsrc_t fil_rsrc =
      make_rsrc(fil, static_cast<size_t>(9) * C * sizeof(T));
  const __amdgpu_buffer_rsrc_t out_rsrc = make_rsrc(out, out_elems * sizeof(T));
  float f[9][V];
#pragma unroll
  for (int t = 0; t < 9; ++t)
    BufVecN<T, V>::load(fil_rsrc,
                     static_cast<unsigned>((FLIP ? 8 - t : t) * C + c) *
                         sizeof(T),
                     f[t]);
  float acc[TH][TW][V];
#pragma unroll
  for (int t = 0; t < TH; ++t)
#pragma unroll
    for (int u = 0; u < TW; ++u)
#pragma unroll
      for (int i = 0; i < V; ++i) acc[t][u][i] = 0.f;
  const int x0 = ox0 * STRIDE - p.pad_cols;
  const int y0 = oy0 * STRIDE - p.pad_rows;
  // Element offset of (n, y0, x0, c); it may lie before the tensor on the
  // border.  Taps outside the image get one fixed out-of-range offset, which
  // the descriptor's range check turns into a zero fill.  (Measured: this
  // select form runs ~15 % faster than or-ing an out-of-range bit into the
  // computed offset.)
  constexpr unsigned kEsz = sizeof(T);
  constexpr int NC = (TW - 1) * STRIDE + 3;
  constexpr int NR = (TH - 1) * STRIDE + 3;
  const int base = ((n * p.in_rows + y0) * p.in_cols + x0) * C + c;
  bool col_ok[NC];
#pragma unroll
  for (int sx = 0; sx < NC; ++sx)
    col_ok[sx] = static_cast<unsigned>(x0 + sx) < static_cast<unsigned>(p.in_cols);
#pragma unroll
  for (int j = 0; j < NR; ++j) {
    const bool row_ok =
        static_cast<unsigned>(y0 + j) < static_cast<unsigned>(p.in_rows);
    float row[NC][V];
#pragma unroll
    for (int sx = 0; sx < NC; ++sx) {
      const unsigned off =
          (row_ok & col_ok[sx])
              ? static_cast<unsigned>(base + (j * p.in_cols + sx) * C) * kEsz
              : kOobOffset;
      BufVecN<T, V>::load(in_rsrc, off, row[sx]);
    }
#pragma unroll
    for (int t = 0; t < TH; ++t) {
      const int r = j - t * STRIDE;  // filter row this input row is for output t
      if (r < 0 || r > 2) continue;
#pragma unroll
      for (int u = 0; u < TW; ++u)
#pragma unroll
        for (int sx = 0; sx < 3; ++sx)
#pragma unroll
          for (int i = 0; i < V; ++i)
            acc[t][u][i] = fmaf(row[u * STRIDE + sx][i], f[r * 3 + sx][i],
                                acc[t][u][i]);
    }
  }
  const int out_base = ((n * p.out_rows + oy0) * p.out_cols + ox0) * C + c;
#pragma unroll
  for (int t = 0; t < TH; ++t) {
#pragma unroll
    for (int u = 0; u < TW; ++u) {
      const unsigned off =
          (oy0 + t < p.out_rows && ox0 + u < p.out_cols)
              ? static_cast<unsigned>(out_base + (t * p.out_cols + u) * C) * kEsz
              : kOobOffset;
      BufVecN<T, V>::store(out_rsrc, off, acc[t][u]);
    }
  }
}

// Forward 3x3, multiplier == 1, fp32, C = 4 * CV with CV in {8, 16, 32}: tall
// strips in which every input vector is loaded by exactly one lane.
//
// The strip kernel above re-loads the window columns its neighbours own (3.0
// vector loads per output at 4 x 2) and leaves the cache to serve them.  Here
// a wave is 64 / CV pixel lanes x CV channel vectors; a lane owns TW
// consecutive output pixels, i.e. STRIDE * TW consecutive input columns (its
// "own" columns: the window centres for stride 1, the first two window
// columns for stride 2), loads only those, and takes the one column to the
// left (stride 1) and to the right of its own range from the neighbouring
// pixel lanes with a cross-lane read (ds_bpermute: the LDS crossbar, no LDS
// memory).  Only the first and last pixel lane of a wave load a halo column
// themselves.  A strip is TH output rows tall and walks down its input rows
// with three (stride 1) or two (stride 2) rows of running sums, storing an
// output row as soon as its third filter row has been added, so the rows that
// two strips share are 2 in TH * STRIDE + 2.  The rows a strip owns are read
// with streaming loads (nobody else reads them); its two halo rows and the
// wave-edge halo columns, which other lanes own, with ordinary ones.
// Work-groups are not remapped to XCDs: consecutive groups then stream
// consecutive runs of the tensor on all XCDs together.  Per output the taps
// are still accumulated in filter-row, filter-column order.  T is float (four
// channels per lane) or half (eight).
//
// 16 bytes of T as raw words, and as floats.
// A loaded vector is split into scalar words through the struct type (the
// whole result bit-cast to uint4): element access on the builtin's own vector
// type has produced wrong code with this compiler.
__device__ inline void load_words(__amdgpu_buffer_rsrc_t r, unsigned off,
                                  unsigned (&v)[4], bool streaming) {
  const uint4 t = __builtin_bit_cast(
      uint4, streaming ? __builtin_amdgcn_raw_buffer_load_b128(r, off, 0, 2)
                       : __builtin_amdgcn_raw_buffer_load_b128(r, off, 0, 0));
  v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
}
template <typename T>
struct Raw16;
template <>
struct Raw16<float> {
  static constexpr int kElems = 4;
  __device__ static void to_float(const unsigned (&r)[4], float (&v)[4]) {
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = __builtin_bit_cast(float, r[i]);
  }
  __device__ static uint4v from_float(const float (&v)[4]) {
    return __builtin_bit_cast(uint4v, make_float4(v[0], v[1], v[2], v[3]));
  }
};
template <>
struct Raw16<_Float16> {
  static constexpr int kElems = 8;
  typedef _Float16 half2v __attribute__((ext_vector_type(2)));
  __device__ static void to_float(const unsigned (&r)[4], float (&v)[8]) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const half2v h = __builtin_bit_cast(half2v, r[i]);
      v[2 * i] = static_cast<float>(h.x);
      v[2 * i + 1] = static_cast<float>(h.y);
    }
  }
  __device__ static uint4v from_float(const float (&v)[8]) {
    typedef _Float16 half8 __attribute__((ext_vector_type(8)));
    half8 t;
#pragma unroll
    for (int i = 0; i < 8; ++i) t[i] = static_cast<_Float16>(v[i]);
    return __builtin_bit_cast(uint4v, t);
  }
};

template <typename T, int STRIDE, int TH, int TW, int CV, bool FLIP>
__global__ void __launch_bounds__(256)
    dw_forward_3x3_tall_kernel(const T* __restrict__ in,
                               const T* __restrict__ fil, T* __restrict__ out,
                               snn_hip_depthwise_params p, int n_strips,
                               int n_wcols, unsigned n_waves) {
  constexpr int V = Raw16<T>::kElems;   // channels per lane: 16 bytes
  constexpr unsigned kEsz = sizeof(T);
  constexpr int PXW = 64 / CV;          // pixel lanes per wave
  constexpr int OWN = STRIDE * TW;      // own input columns per lane
  constexpr int A = STRIDE == 1 ? 1 : 0;  // own range starts A columns right of
                                          // the first window column
  constexpr int NR = (TH - 1) * STRIDE + 3;
  constexpr int LIVE = STRIDE == 1 ? 3 : 2;  // output rows with open sums
  const unsigned w = blockIdx.x * 4u + (threadIdx.x >> 6);
  if (w >= n_waves) return;  // whole waves only: the cross-lane reads below
                             // need every lane of a live wave
  const int lane = threadIdx.x & 63;
  const int cvi = lane % CV, pl = lane / CV;
  const int wcol = static_cast<int>(w % static_cast<unsigned>(n_wcols));
  const unsigned rest = w / static_cast<unsigned>(n_wcols);
  const int strip = static_cast<int>(rest % static_cast<unsigned>(n_strips));
  const int n = static_cast<int>(rest / static_cast<unsigned>(n_strips));
  const int C = p.channels, c = cvi * V;
  const size_t in_elems =
      static_cast<size_t>(p.batch) * p.in_rows * p.in_cols * C;
  const size_t out_elems =
      static_cast<size_t>(p.batch) * p.out_rows * p.out_cols * C;
  const __amdgpu_buffer_rsrc_t in_rsrc = make_rsrc(in, in_elems * kEsz);
  const __amdgpu_buffer_rsrc_t fil_rsrc =
      make_rsrc(fil, static_cast<size_t>(9) * C * kEsz);
  const __amdgpu_buffer_rsrc_t out_rsrc = make_rsrc(out, out_elems * kEsz);
  float f[9][V];
#pragma unroll
  for (int t = 0; t < 9; ++t) {
    unsigned words[4];
    load_words(fil_rsrc,
               static_cast<unsigned>((FLIP ? 8 - t : t) * C + c) * kEsz, words,
               false);
    Raw16<T>::to_float(words, f[t]);
  }
  const int oy0 = strip * TH;
  const int ox0 = (wcol * PXW + pl) * TW;  // first own output pixel
  const int col0 = STRIDE * ox0 - p.pad_cols + A;  // first own input column
  const int y0 = STRIDE * oy0 - p.pad_rows;        // first input row
  // the wave's halo columns, loaded by its first / last pixel lane only
  const int xl = STRIDE * (wcol * PXW * TW) - p.pad_cols + A - 1;
  const int xr = STRIDE * ((wcol + 1) * PXW * TW) - p.pad_cols + A;
  const bool first = pl == 0, last = pl == PXW - 1;
  const bool l_ok = STRIDE == 1 && first &&
                    static_cast<unsigned>(xl) < static_cast<unsigned>(p.in_cols);
  const bool r_ok =
      last && static_cast<unsigned>(xr) < static_cast<unsigned>(p.in_cols);
  bool own_ok[OWN];
#pragma unroll
  for (int k = 0; k < OWN; ++k)
    own_ok[k] = static_cast<unsigned>(col0 + k) <
                static_cast<unsigned>(p.in_cols);
  // element offset of (n, y0, column 0, c)
  const int row0 = (n * p.in_rows + y0) * p.in_cols * C + c;
  const int rstride = p.in_cols * C;
  const int src_l = (lane - CV) * 4, src_r = (lane + CV) * 4;

  unsigned own[NR][OWN][4], hl[NR][4], hr[NR][4];
#pragma unroll
  for (int j = 0; j < NR; ++j) {
    const bool row_ok =
        static_cast<unsigned>(y0 + j) < static_cast<unsigned>(p.in_rows);
    // rows A .. A + STRIDE * TH - 1 of the strip are read by this strip only
    const bool mine = j >= A && j < A + STRIDE * TH;
#pragma unroll
    for (int k = 0; k < OWN; ++k)
      load_words(
          in_rsrc,
          (row_ok && own_ok[k])
              ? static_cast<unsigned>(row0 + j * rstride + (col0 + k) * C) * kEsz
              : kOobOffset,
          own[j][k], mine);
    if (STRIDE == 1)
      load_words(in_rsrc,
                 (row_ok && l_ok)
                     ? static_cast<unsigned>(row0 + j * rstride + xl * C) * kEsz
                     : kOobOffset,
                 hl[j], false);
    load_words(in_rsrc,
               (row_ok && r_ok)
                   ? static_cast<unsigned>(row0 + j * rstride + xr * C) * kEsz
                   : kOobOffset,
               hr[j], false);
  }

  float acc[LIVE][TW][V];
#pragma unroll
  for (int j = 0; j < NR; ++j) {
    // win[k + 1] is input column col0 + k, k = -1 .. OWN.  The neighbours'
    // columns cross the lanes as raw words (half as many exchanges for T =
    // half as exchanging the converted values would take).
    float win[OWN + 2][V];
    {
      unsigned left[4], right[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        if (STRIDE == 1) {
          const unsigned from_left =
              static_cast<unsigned>(__builtin_amdgcn_ds_bpermute(
                  src_l, static_cast<int>(own[j][OWN - 1][i])));
          left[i] = first ? hl[j][i] : from_left;
        } else {
          left[i] = 0u;
        }
        const unsigned from_right =
            static_cast<unsigned>(__builtin_amdgcn_ds_bpermute(
                src_r, static_cast<int>(own[j][0][i])));
        right[i] = last ? hr[j][i] : from_right;
      }
      Raw16<T>::to_float(left, win[0]);
      Raw16<T>::to_float(right, win[OWN + 1]);
#pragma unroll
      for (int k = 0; k < OWN; ++k) Raw16<T>::to_float(own[j][k], win[k + 1]);
    }
    // input row j is filter row r of output row t = (j - r) / STRIDE; the
    // older output row first
#pragma unroll
    for (int r = 2; r >= 0; --r) {
      if (j - r < 0 || (j - r) % STRIDE != 0) continue;
      const int t = (j - r) / STRIDE;
      if (t >= TH) continue;
#pragma unroll
      for (int u = 0; u < TW; ++u) {
#pragma unroll
        for (int i = 0; i < V; ++i) {
          float a = r == 0 ? 0.f : acc[t % LIVE][u][i];
#pragma unroll
          for (int sx = 0; sx < 3; ++sx)
            a = fmaf(win[STRIDE * u + sx - A + 1][i], f[r * 3 + sx][i], a);
          acc[t % LIVE][u][i] = a;
        }
      }
      if (r == 2) {
#pragma unroll
        for (int u = 0; u < TW; ++u) {
          const bool ok = oy0 + t < p.out_rows && ox0 + u < p.out_cols;
          __builtin_amdgcn_raw_buffer_store_b128(
              Raw16<T>::from_float(acc[t % LIVE][u]), out_rsrc,
              ok ? static_cast<unsigned>(
                       ((n * p.out_rows + oy0 + t) * p.out_cols + ox0 + u) * C +
                       c) * kEsz
                 : kOobOffset,
              0, kStoreAux);
        }
      }
    }
  }
}

// Forward, any multiplier / channel count: one lane per output element.
template <typename T>
__global__ void __launch_bounds__(256)
    dw_forward_scalar_kernel(const T* __restrict__ in,
                             const T* __restrict__ fil, T* __restrict__ out,
                             snn_hip_depthwise_params p, size_t n_out) {
  const size_t idx = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (idx >= n_out) return;
  const int C = p.channels, M = p.channel_multiplier;
  const int cm = static_cast<int>(idx % (static_cast<size_t>(C) * M));
  const int c = cm / M, j = cm % M;
  size_t pix = idx / (static_cast<size_t>(C) * M);
  const int ox = static_cast<int>(pix % p.out_cols);
  pix /= p.out_cols;
  const int oy = static_cast<int>(pix % p.out_rows);
  const int n = static_cast<int>(pix / p.out_rows);
  const T* in_n = in + static_cast<size_t>(n) * p.in_rows * p.in_cols * C + c;
  float acc = 0.f;
  for (int r = 0; r < p.window_rows; ++r) {
    const int y = oy * p.stride_rows - p.pad_rows + r;
    if (y < 0 || y >= p.in_rows) continue;
    for (int s = 0; s < p.window_cols; ++s) {
      const int x = ox * p.stride_cols - p.pad_cols + s;
      if (x < 0 || x >= p.in_cols) continue;
      acc = fmaf(
          Elem<T>::load(in_n + (static_cast<size_t>(y) * p.in_cols + x) * C),
          Elem<T>::load(fil +
                        (static_cast<size_t>(r * p.window_cols + s) * C + c) * M +
                        j),
          acc);
    }
  }
  out[idx] = Elem<T>::from_float(acc);
}

// Input backprop: one lane per dX element (n, y, x, c).
template <typename T>
__global__ void __launch_bounds__(256)
    dw_input_backprop_kernel(const T* __restrict__ dy,
                             const T* __restrict__ fil, T* __restrict__ dx,
                             snn_hip_depthwise_params p, size_t n_out) {
  const size_t idx = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (idx >= n_out) return;
  const int C = p.channels, M = p.channel_multiplier;
  const int c = static_cast<int>(idx % C);
  size_t pix = idx / C;
  const int x = static_cast<int>(pix % p.in_cols);
  pix /= p.in_cols;
  const int y = static_cast<int>(pix % p.in_rows);
  const int n = static_cast<int>(pix / p.in_rows);
  const T* dy_n =
      dy + static_cast<size_t>(n) * p.out_rows * p.out_cols * C * M;
  float acc = 0.f;
  for (int r = 0; r < p.window_rows; ++r) {
    const int ty = y + p.pad_rows - r;
    if (ty < 0 || ty % p.stride_rows) continue;
    const int oy = ty / p.stride_rows;
    if (oy >= p.out_rows) continue;
    for (int s = 0; s < p.window_cols; ++s) {
      const int tx = x + p.pad_cols - s;
      if (tx < 0 || tx % p.stride_cols) continue;
      const int ox = tx / p.stride_cols;
      if (ox >= p.out_cols) continue;
      const T* gp =
          dy_n + ((static_cast<size_t>(oy) * p.out_cols + ox) * C + c) * M;
      const T* fp =
          fil + (static_cast<size_t>(r * p.window_cols + s) * C + c) * M;
      for (int j = 0; j < M; ++j) {
        acc = fmaf(Elem<T>::load(gp + j), Elem<T>::load(fp + j), acc);
      }
    }
  }
  dx[idx] = Elem<T>::from_float(acc);
}

// Input backprop, multiplier == 1, C % 4 == 0, any window / stride: one lane
// per four channels of a dX pixel; for stride 2 at most two taps per axis
// reach a pixel.
template <typename T>
__global__ void __launch_bounds__(256)
    dw_input_backprop_vec4_kernel(const T* __restrict__ dy,
                                  const T* __restrict__ fil,
                                  T* __restrict__ dx,
                                  snn_hip_depthwise_params p, unsigned n_vec) {
  const unsigned idx = gemm::xcd_remap(blockIdx.x, gridDim.x) * 256u +
                       threadIdx.x;
  if (idx >= n_vec) return;
  const int C = p.channels;
  const unsigned cv = static_cast<unsigned>(C) / 4u;
  const int c = static_cast<int>(idx % cv) * 4;
  unsigned pix = idx / cv;
  const int x = static_cast<int>(pix % static_cast<unsigned>(p.in_cols));
  pix /= static_cast<unsigned>(p.in_cols);
  const int y = static_cast<int>(pix % static_cast<unsigned>(p.in_rows));
  const int n = static_cast<int>(pix / static_cast<unsigned>(p.in_rows));
  const size_t dy_elems =
      static_cast<size_t>(p.batch) * p.out_rows * p.out_cols * C;
  const size_t dx_elems =
      static_cast<size_t>(p.batch) * p.in_rows * p.in_cols * C;
  const __amdgpu_buffer_rsrc_t dy_rsrc = make_rsrc(dy, dy_elems * sizeof(T));
  const __amdgpu_buffer_rsrc_t fil_rsrc = make_rsrc(
      fil, static_cast<size_t>(p.window_rows) * p.window_cols * C * sizeof(T));
  const __amdgpu_buffer_rsrc_t dx_rsrc = make_rsrc(dx, dx_elems * sizeof(T));
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  // first tap row / column whose offset from (y + pad) is a multiple of the
  // stride
  const int ty0 = y + p.pad_rows, tx0 = x + p.pad_cols;
  for (int r = ty0 % p.stride_rows; r < p.window_rows; r += p.stride_rows) {
    const int oy = (ty0 - r) / p.stride_rows;
    if (ty0 - r < 0 || oy >= p.out_rows) continue;
    for (int sc = tx0 % p.stride_cols; sc < p.window_cols;
         sc += p.stride_cols) {
      const int ox = (tx0 - sc) / p.stride_cols;
      if (tx0 - sc < 0 || ox >= p.out_cols) continue;
      float g[4], f[4];
      BufVec4<T>::load(
          dy_rsrc,
          static_cast<unsigned>(((n * p.out_rows + oy) * p.out_cols + ox) * C +
                                c) * sizeof(T),
          g);
      BufVec4<T>::load(
          fil_rsrc,
          static_cast<unsigned>((r * p.window_cols + sc) * C + c) * sizeof(T),
          f);
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[i] = fmaf(g[i], f[i], acc[i]);
    }
  }
  BufVec4<T>::store(dx_rsrc, idx * 4u * static_cast<unsigned>(sizeof(T)), acc);
}

// Input backprop, 3x3 stride 2, multiplier == 1, four channels per lane.
// In padded coordinates t = y + pad a dX pixel with even t takes filter rows
// 0 and 2 (from dY rows t / 2 and t / 2 - 1) and one with odd t takes row 1
// (from dY row t / 2); columns alike.  A lane owns the 2 x 2 dX pixels of
// TH consecutive block rows of one block column: four dY vectors feed the
// four pixels of a block, two of them carried over from the block row above,
// and the nine filter taps stay in registers.  Every dX pixel still adds its
// taps in filter-row, filter-column order.
template <typename T, int TH>
__global__ void __launch_bounds__(256)
    dw_input_backprop_3x3_s2_kernel(const T* __restrict__ dy,
                                    const T* __restrict__ fil,
                                    T* __restrict__ dx,
                                    snn_hip_depthwise_params p, int n_bcols,
                                    int n_strips, unsigned n_items) {
  const unsigned idx = blockIdx.x * 256u + threadIdx.x;
  if (idx >= n_items) return;
  const int C = p.channels;
  const unsigned cv = static_cast<unsigned>(C) / 4u;
  const int c = static_cast<int>(idx % cv) * 4;
  unsigned t = idx / cv;
  const int bc = static_cast<int>(t % static_cast<unsigned>(n_bcols)) +
                 p.pad_cols / 2;
  t /= static_cast<unsigned>(n_bcols);
  const int br0 = static_cast<int>(t % static_cast<unsigned>(n_strips)) * TH +
                  p.pad_rows / 2;
  const int n = static_cast<int>(t / static_cast<unsigned>(n_strips));
  const size_t dy_elems =
      static_cast<size_t>(p.batch) * p.out_rows * p.out_cols * C;
  const size_t dx_elems =
      static_cast<size_t>(p.batch) * p.in_rows * p.in_cols * C;
  const __amdgpu_buffer_rsrc_t dy_rsrc = make_rsrc(dy, dy_elems * sizeof(T));
  const __amdgpu_buffer_rsrc_t fil_rsrc =
      make_rsrc(fil, static_cast<size_t>(9) * C * sizeof(T));
  const __amdgpu_buffer_rsrc_t dx_rsrc = make_rsrc(dx, dx_elems * sizeof(T));
  float f[9][4];
#pragma unroll
  for (int k = 0; k < 9; ++k)
    BufVec4<T>::load(fil_rsrc,
                     static_cast<unsigned>(k * C + c) * sizeof(T), f[k]);
  // dY columns bc - 1 and bc of one dY row; out of range reads zeros
  const bool col_ok[2] = {bc >= 1 && bc - 1 < p.out_cols, bc < p.out_cols};
  auto load_row = [&](int oy, float (&g)[2][4]) {
    const bool row_ok =
        static_cast<unsigned>(oy) < static_cast<unsigned>(p.out_rows);
    const unsigned base =
        static_cast<unsigned>(((n * p.out_rows + oy) * p.out_cols + bc - 1) *
                                  C + c) * sizeof(T);
#pragma unroll
    for (int j = 0; j < 2; ++j)
      BufVec4<T>::load(dy_rsrc,
                       (row_ok && col_ok[j])
                           ? base + static_cast<unsigned>(j * C) * sizeof(T)
                           : kOobOffset,
                       g[j]);
  };
  // dX pixel (2 * br - pad + i, 2 * bc - pad + j) of the current block
  const int x0 = 2 * bc - p.pad_cols;
  const bool x_ok[2] = {
      static_cast<unsigned>(x0) < static_cast<unsigned>(p.in_cols),
      static_cast<unsigned>(x0 + 1) < static_cast<unsigned>(p.in_cols)};
  float above[2][4], here[2][4];
  load_row(br0 - 1, above);
#pragma unroll
  for (int i = 0; i < TH; ++i) {
    const int br = br0 + i;
    load_row(br, here);
    float even_even[4], even_odd[4], odd_even[4], odd_odd[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      // taps in (r, s) order: (0,0) (0,2) (2,0) (2,2)
      float v = here[1][e] * f[0][e];
      v = fmaf(here[0][e], f[2][e], v);
      v = fmaf(above[1][e], f[6][e], v);
      even_even[e] = fmaf(above[0][e], f[8][e], v);
      // (0,1) (2,1)
      even_odd[e] = fmaf(above[1][e], f[7][e], here[1][e] * f[1][e]);
      // (1,0) (1,2)
      odd_even[e] = fmaf(here[0][e], f[5][e], here[1][e] * f[3][e]);
      // (1,1)
      odd_odd[e] = here[1][e] * f[4][e];
    }
    const int y0 = 2 * br - p.pad_rows;
    const bool y_ok[2] = {
        static_cast<unsigned>(y0) < static_cast<unsigned>(p.in_rows),
        static_cast<unsigned>(y0 + 1) < static_cast<unsigned>(p.in_rows)};
    const unsigned base =
        static_cast<unsigned>(((n * p.in_rows + y0) * p.in_cols + x0) * C + c) *
        sizeof(T);
    const unsigned row_bytes =
        static_cast<unsigned>(p.in_cols * C) * sizeof(T);
    const unsigned col_bytes = static_cast<unsigned>(C) * sizeof(T);
    BufVec4<T>::store(dx_rsrc, (y_ok[0] && x_ok[0]) ? base : kOobOffset,
                      even_even);
    BufVec4<T>::store(dx_rsrc,
                      (y_ok[0] && x_ok[1]) ? base + col_bytes : kOobOffset,
                      even_odd);
    BufVec4<T>::store(dx_rsrc,
                      (y_ok[1] && x_ok[0]) ? base + row_bytes : kOobOffset,
                      odd_even);
    BufVec4<T>::store(
        dx_rsrc,
        (y_ok[1] && x_ok[1]) ? base + row_bytes + col_bytes : kOobOffset,
        odd_odd);
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int e = 0; e < 4; ++e) above[j][e] = here[j][e];
  }
}

// Filter backprop, 3x3, multiplier == 1, C % 4 == 0.  A work-group covers
// `cvw` channel vectors x (256 / cvw) pixels at a time and walks a range of
// output pixels; each lane keeps the 9 x 4 partial sums of its channels, the
// pixel lanes are then added up through LDS and the result goes to the
// zero-filled dF with float atomics.  fp32 only (float atomics).
constexpr int kDwFilbkThreads = 256;

__global__ void __launch_bounds__(kDwFilbkThreads)
    dw_filter_backprop_3x3_kernel(const float* __restrict__ in,
                                  const float* __restrict__ dy,
                                  float* __restrict__ dw,
                                  snn_hip_depthwise_params p, int cvw,
                                  int pixels_per_group) {
  __shared__ float partial[kDwFilbkThreads][37];
  const int C = p.channels;
  const int tid = threadIdx.x;
  const int cl = tid % cvw;          // channel vector inside the group
  const int pl = tid / cvw;          // pixel lane
  const int n_pl = kDwFilbkThreads / cvw;
  const int c = (blockIdx.y * cvw + cl) * 4;
  const int n_pix = p.batch * p.out_rows * p.out_cols;
  const int pix_begin = blockIdx.x * pixels_per_group;
  const int pix_end = min(n_pix, pix_begin + pixels_per_group);
  const size_t in_elems =
      static_cast<size_t>(p.batch) * p.in_rows * p.in_cols * C;
  const size_t dy_elems = static_cast<size_t>(n_pix) * C;
  const __amdgpu_buffer_rsrc_t in_rsrc = make_rsrc(in, in_elems * 4);
  const __amdgpu_buffer_rsrc_t dy_rsrc = make_rsrc(dy, dy_elems * 4);
  float acc[9][4];
#pragma unroll
  for (int t = 0; t < 9; ++t)
#pragma unroll
    for (int i = 0; i < 4; ++i) acc[t][i] = 0.f;
  if (c < C) {
    for (int pix = pix_begin + pl; pix < pix_end; pix += n_pl) {
      const int ox = pix % p.out_cols;
      const int t2 = pix / p.out_cols;
      const int oy = t2 % p.out_rows;
      const int n = t2 / p.out_rows;
      const int y0 = oy * p.stride_rows - p.pad_rows;
      const int x0 = ox * p.stride_cols - p.pad_cols;
      float g[4];
      BufVec4<float>::load(dy_rsrc, static_cast<unsigned>(pix * C + c) * 4u, g);
      const int base = ((n * p.in_rows + y0) * p.in_cols + x0) * C + c;
#pragma unroll
      for (int r = 0; r < 3; ++r) {
        const bool row_ok =
            static_cast<unsigned>(y0 + r) < static_cast<unsigned>(p.in_rows);
#pragma unroll
        for (int sc = 0; sc < 3; ++sc) {
          const bool ok = row_ok & (static_cast<unsigned>(x0 + sc) <
                                    static_cast<unsigned>(p.in_cols));
          float xv[4];
          BufVec4<float>::load(
              in_rsrc,
              ok ? static_cast<unsigned>(base + (r * p.in_cols + sc) * C) * 4u
                 : kOobOffset,
              xv);
#pragma unroll
          for (int i = 0; i < 4; ++i)
            acc[r * 3 + sc][i] = fmaf(xv[i], g[i], acc[r * 3 + sc][i]);
        }
      }
    }
  }
#pragma unroll
  for (int t = 0; t < 9; ++t)
#pragma unroll
    for (int i = 0; i < 4; ++i) partial[tid][t * 4 + i] = acc[t][i];
  __syncthreads();
  // lane e of the first cvw * 36 adds up one (channel vector, tap, component)
  for (int e = tid; e < cvw * 36; e += kDwFilbkThreads) {
    const int ecl = e % cvw, comp = e / cvw;  // comp = tap * 4 + i
    float sum = 0.f;
    for (int q = 0; q < n_pl; ++q) sum += partial[q * cvw + ecl][comp];
    const int ch = (blockIdx.y * cvw + ecl) * 4 + (comp & 3);
    if (ch < C) atomicAdd(dw + (comp >> 2) * C + ch, sum);
  }
}

// The same reduction with the input window kept in registers: a pixel lane
// walks TH consecutive output rows of TW adjacent output columns and loads
// every input row of that strip once, so two stride-1 output pixels cost
// 4 + 2 vector loads instead of 20.  Strips are numbered column block
// fastest, (image, row block, column block), and dealt to the pixel lanes in
// that order; rows and columns past the end of the image read zeros through
// the buffer range check and add nothing.  The pixel lanes of a wave are added
// up across lanes, the four waves through LDS.
template <int STRIDE, int TH, int TW, int AHEAD, typename T = float>
__global__ void __launch_bounds__(kDwFilbkThreads)
    dw_filter_backprop_3x3_strip_kernel(const T* __restrict__ in,
                                        const T* __restrict__ dy,
                                        float* __restrict__ dw,
                                        float* __restrict__ part,
                                        snn_hip_depthwise_params p, int cvw,
                                        int strips_per_group, int n_strips,
                                        int n_row_blocks, int n_col_blocks) {
  constexpr unsigned kEsz = sizeof(T);
  // A strip is TH output rows of TW adjacent output columns, so an input row
  // costs NC column loads for TW outputs.  The loads of output row i + AHEAD
  // are issued before the products of row i.
  constexpr int NC = (TW - 1) * STRIDE + 3;  // input columns of a strip
  constexpr int RING = AHEAD * STRIDE + 3;   // input rows alive at once
  constexpr int GRING = AHEAD + 1;           // dY rows alive at once
  __shared__ float partial[4][32][37];       // [wave][channel vector][tap * 4 + i]
  const int C = p.channels;
  const int tid = threadIdx.x;
  const int cl = tid % cvw;
  const int pl = tid / cvw;
  const int n_pl = kDwFilbkThreads / cvw;
  const int c = (blockIdx.y * cvw + cl) * 4;
  const int strip_begin = blockIdx.x * strips_per_group;
  const int strip_end = min(n_strips, strip_begin + strips_per_group);
  const size_t in_elems =
      static_cast<size_t>(p.batch) * p.in_rows * p.in_cols * C;
  const size_t dy_elems =
      static_cast<size_t>(p.batch) * p.out_rows * p.out_cols * C;
  const __amdgpu_buffer_rsrc_t in_rsrc = make_rsrc(in, in_elems * kEsz);
  const __amdgpu_buffer_rsrc_t dy_rsrc = make_rsrc(dy, dy_elems * kEsz);
  float acc[9][4];
#pragma unroll
  for (int t = 0; t < 9; ++t)
#pragma unroll
    for (int i = 0; i < 4; ++i) acc[t][i] = 0.f;
  if (c < C) {
    for (int strip = strip_begin + pl; strip < strip_end; strip += n_pl) {
      const int ox = (strip % n_col_blocks) * TW;
      const int t2 = strip / n_col_blocks;
      const int rb = t2 % n_row_blocks;
      const int n = t2 / n_row_blocks;
      const int oy0 = rb * TH;
      const int y0 = oy0 * STRIDE - p.pad_rows;
      const int x0 = ox * STRIDE - p.pad_cols;
      // byte offsets of the strip's input columns in row 0 of the image, or
      // out of range for a padding column
      unsigned col_off[NC];
#pragma unroll
      for (int sc = 0; sc < NC; ++sc)
        col_off[sc] = static_cast<unsigned>(x0 + sc) <
                              static_cast<unsigned>(p.in_cols)
                          ? static_cast<unsigned>((x0 + sc) * C + c) * kEsz
                          : kOobOffset;
      const unsigned image_off =
          static_cast<unsigned>(n * p.in_rows * p.in_cols * C) * kEsz;
      const unsigned row_bytes = static_cast<unsigned>(p.in_cols * C) * kEsz;
      float win[RING][NC][4];
      // (Offsets of rows and columns outside the image are made out of range
      // with mask arithmetic, not with a conditional: the compiler turns a
      // per-lane condition around these loads into two branches that load
      // into the same registers, and has to wait for every load in flight
      // between them -- which undid the row of loads issued ahead.)
      auto load_row = [&](int rel, float (&dst)[NC][4]) {
        const int y = y0 + rel;
        const unsigned bad_row =
            0u - static_cast<unsigned>(static_cast<unsigned>(y) >=
                                       static_cast<unsigned>(p.in_rows));
        const unsigned base =
            image_off + static_cast<unsigned>(y) * row_bytes;
#pragma unroll
        for (int sc = 0; sc < NC; ++sc) {
          const unsigned bad =
              bad_row |
              (0u - static_cast<unsigned>(col_off[sc] == kOobOffset));
          BufVec4<T>::load(
              in_rsrc, ((base + col_off[sc]) & ~bad) | (kOobOffset & bad),
              dst[sc]);
        }
      };
      const unsigned dy_off0 =
          static_cast<unsigned>(((n * p.out_rows + oy0) * p.out_cols + ox) * C +
                                c) * kEsz;
      const unsigned dy_row_bytes = static_cast<unsigned>(p.out_cols * C) * kEsz;
      float g[GRING][TW][4];
      // the input rows output row i adds that row i - 1 lacked, and its dY
      auto load_out_row = [&](int i) {
#pragma unroll
        for (int rel = 3 - STRIDE; rel < 3; ++rel)
          load_row(i * STRIDE + rel, win[(i * STRIDE + rel) % RING]);
#pragma unroll
        for (int tw = 0; tw < TW; ++tw) {
          const unsigned bad =
              0u - static_cast<unsigned>(oy0 + i >= p.out_rows ||
                                         ox + tw >= p.out_cols);
          BufVec4<T>::load(
              dy_rsrc,
              ((dy_off0 + static_cast<unsigned>(i) * dy_row_bytes +
                static_cast<unsigned>(tw * C) * kEsz) & ~bad) |
                  (kOobOffset & bad),
              g[i % GRING][tw]);
        }
      };
#pragma unroll
      for (int rel = 0; rel < 3 - STRIDE; ++rel) load_row(rel, win[rel % RING]);
#pragma unroll
      for (int i = 0; i < AHEAD && i < TH; ++i) load_out_row(i);
#pragma unroll
      for (int i = 0; i < TH; ++i) {
        if (i + AHEAD < TH) load_out_row(i + AHEAD);
#pragma unroll
        for (int tw = 0; tw < TW; ++tw) {
          // (a strip may run past the last output row or column: nothing to
          // add there, whatever the input under it holds)
          if (oy0 + i < p.out_rows && ox + tw < p.out_cols) {
#pragma unroll
            for (int r = 0; r < 3; ++r)
#pragma unroll
              for (int sc = 0; sc < 3; ++sc)
#pragma unroll
                for (int e = 0; e < 4; ++e)
                  acc[r * 3 + sc][e] =
                      fmaf(win[(i * STRIDE + r) % RING][tw * STRIDE + sc][e],
                           g[i % GRING][tw][e], acc[r * 3 + sc][e]);
          }
        }
      }
    }
  }
  // The lanes of a wave that share a channel vector are l, l ^ cvw,
  // l ^ 2 cvw, ...: add them up across lanes, then the four waves through LDS.
  for (int m = cvw; m < 64; m <<= 1) {
#pragma unroll
    for (int t = 0; t < 9; ++t)
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[t][i] += __shfl_xor(acc[t][i], m);
  }
  const int lane = tid & 63, wave = tid >> 6;
  if (lane < cvw) {
#pragma unroll
    for (int t = 0; t < 9; ++t)
#pragma unroll
      for (int i = 0; i < 4; ++i) partial[wave][lane][t * 4 + i] = acc[t][i];
  }
  __syncthreads();
  // lane e of the first cvw * 36 adds up one (channel vector, tap, component)
  for (int e = tid; e < cvw * 36; e += kDwFilbkThreads) {
    const int ecl = e % cvw, comp = e / cvw;  // comp = tap * 4 + i
    const float sum = (partial[0][ecl][comp] + partial[1][ecl][comp]) +
                      (partial[2][ecl][comp] + partial[3][ecl][comp]);
    const int ch = (blockIdx.y * cvw + ecl) * 4 + (comp & 3);
    if (ch >= C) continue;
    if (part != nullptr) {
      part[static_cast<size_t>(blockIdx.x) * 9 * C + (comp >> 2) * C + ch] =
          sum;
      // the kernel that adds the partial filters up expects dF zero-filled
      if (blockIdx.x == 0) dw[(comp >> 2) * C + ch] = 0.f;
    } else {
      atomicAdd(dw + (comp >> 2) * C + ch, sum);
    }
  }
}

// dF += the work-groups' partial filters part[group][e], four elements per
// lane.  blockIdx.y and the four waves of a work-group split the groups into
// gridDim.y * 4 slices; the launcher sizes gridDim.y so that a lane has at most
// kDwFilbkReduceLoads groups to add, and their loads are all issued before the
// first addition.  The waves combine through LDS and one float atomic per
// element and work-group goes to dF, which the strip kernel has zero-filled.
constexpr int kDwFilbkReduceLoads = 8;

__global__ void __launch_bounds__(256)
    dw_filbk_reduce_kernel(const float4* __restrict__ part,
                           float* __restrict__ dw, int n_vec, int n_groups) {
  __shared__ float4 sums[4][64];
  const int lane = threadIdx.x & 63, sub = threadIdx.x >> 6;
  const int v = blockIdx.x * 64 + lane;
  const int n_slices = gridDim.y * 4;
  float4 a = make_float4(0.f, 0.f, 0.f, 0.f);
  if (v < n_vec) {
    for (int g0 = blockIdx.y * 4 + sub; g0 < n_groups;
         g0 += kDwFilbkReduceLoads * n_slices) {
      float4 x[kDwFilbkReduceLoads];
#pragma unroll
      for (int k = 0; k < kDwFilbkReduceLoads; ++k) {
        // a group index past the end re-reads the last group and is not added
        const int g = min(g0 + k * n_slices, n_groups - 1);
        x[k] = part[static_cast<size_t>(g) * n_vec + v];
      }
#pragma unroll
      for (int k = 0; k < kDwFilbkReduceLoads; ++k) {
        if (g0 + k * n_slices < n_groups)
          a = make_float4(a.x + x[k].x, a.y + x[k].y, a.z + x[k].z,
                          a.w + x[k].w);
      }
    }
  }
  sums[sub][lane] = a;
  __syncthreads();
  if (sub == 0 && v < n_vec) {
    const float4 s0 = sums[0][lane], s1 = sums[1][lane], s2 = sums[2][lane],
                 s3 = sums[3][lane];
    atomicAdd(dw + 4 * v + 0, (s0.x + s1.x) + (s2.x + s3.x));
    atomicAdd(dw + 4 * v + 1, (s0.y + s1.y) + (s2.y + s3.y));
    atomicAdd(dw + 4 * v + 2, (s0.z + s1.z) + (s2.z + s3.z));
    atomicAdd(dw + 4 * v + 3, (s0.w + s1.w) + (s2.w + s3.w));
  }
}

__global__ void __launch_bounds__(256)
    dw_zero_kernel(float* __restrict__ p, int n) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i < n) p[i] = 0.f;
}

constexpr int kStrip = 64;   // (channel, multiplier) pairs per work-group
constexpr int kSlices = 4;   // waves splitting the batch*rows*cols reduction

// Filter backprop: one work-group per filter tap (r, s) and strip of 64
// flattened (c, j) outputs; the four waves split the reduction over every
// output pixel and combine through LDS.
template <typename T>
__global__ void __launch_bounds__(kStrip* kSlices)
    dw_filter_backprop_kernel(const T* __restrict__ in,
                              const T* __restrict__ dy, T* __restrict__ dw,
                              snn_hip_depthwise_params p) {
  __shared__ float partial[kSlices][kStrip];
  const int C = p.channels, M = p.channel_multiplier;
  const int CM = C * M;
  const int lane = threadIdx.x % kStrip;
  const int slice = threadIdx.x / kStrip;
  const int cm = blockIdx.y * kStrip + lane;
  const int s = blockIdx.x % p.window_cols;
  const int r = blockIdx.x / p.window_cols;
  const int c = cm / M;
  const int n_pix = p.batch * p.out_rows * p.out_cols;
  float acc = 0.f;
  if (cm < CM) {
    for (int pix = slice; pix < n_pix; pix += kSlices) {
      const int ox = pix % p.out_cols;
      const int t = pix / p.out_cols;
      const int oy = t % p.out_rows;
      const int n = t / p.out_rows;
      const int y = oy * p.stride_rows - p.pad_rows + r;
      const int x = ox * p.stride_cols - p.pad_cols + s;
      if (y < 0 || y >= p.in_rows || x < 0 || x >= p.in_cols) continue;
      const float xv = Elem<T>::load(
          in + ((static_cast<size_t>(n) * p.in_rows + y) * p.in_cols + x) * C +
          c);
      const float gv = Elem<T>::load(dy + static_cast<size_t>(pix) * CM + cm);
      acc = fmaf(xv, gv, acc);
    }
  }
  partial[slice][lane] = acc;
  __syncthreads();
  if (slice == 0 && cm < CM) {
    float sum = partial[0][lane];
    for (int i = 1; i < kSlices; ++i) sum += partial[i][lane];
    dw[static_cast<size_t>(blockIdx.x) * CM + cm] = Elem<T>::from_float(sum);
  }
}

// The same with the output pixels also split over work-groups (blockIdx.z:
// `per_chunk` consecutive pixels each), for launches whose (tap, strip) pairs
// alone would leave most of the GPU idle: a slice walks its run of pixels
// with (image, row, column) advanced incrementally, and the work-groups' sums
// meet in the zero-filled fp32 buffer `acc` through float atomics.
template <typename T>
__global__ void __launch_bounds__(kStrip* kSlices)
    dw_filter_backprop_split_kernel(const T* __restrict__ in,
                                    const T* __restrict__ dy,
                                    float* __restrict__ acc,
                                    snn_hip_depthwise_params p, int per_chunk) {
  __shared__ float partial[kSlices][kStrip];
  const int C = p.channels, M = p.channel_multiplier;
  const int CM = C * M;
  const int lane = threadIdx.x % kStrip;
  const int slice = threadIdx.x / kStrip;
  const int cm = blockIdx.y * kStrip + lane;
  const int s = blockIdx.x % p.window_cols;
  const int r = blockIdx.x / p.window_cols;
  const int c = cm / M;
  const int n_pix = p.batch * p.out_rows * p.out_cols;
  const int begin = blockIdx.z * per_chunk;
  const int end = min(n_pix, begin + per_chunk);
  const int per_slice = (end - begin + kSlices - 1) / kSlices;
  const int first = begin + slice * per_slice;
  const int last = min(end, first + per_slice);
  float sum = 0.f;
  if (cm < CM && first < last) {
    int ox = first % p.out_cols;
    const int t = first / p.out_cols;
    int oy = t % p.out_rows;
    int n = t / p.out_rows;
#pragma unroll 4
    for (int pix = first; pix < last; ++pix) {
      const int y = oy * p.stride_rows - p.pad_rows + r;
      const int x = ox * p.stride_cols - p.pad_cols + s;
      if (y >= 0 && y < p.in_rows && x >= 0 && x < p.in_cols) {
        const float xv = Elem<T>::load(
            in + ((static_cast<size_t>(n) * p.in_rows + y) * p.in_cols + x) * C +
            c);
        const float gv = Elem<T>::load(dy + static_cast<size_t>(pix) * CM + cm);
        sum = fmaf(xv, gv, sum);
      }
      if (++ox == p.out_cols) {
        ox = 0;
        if (++oy == p.out_rows) {
          oy = 0;
          ++n;
        }
      }
    }
  }
  partial[slice][lane] = sum;
  __syncthreads();
  if (slice == 0 && cm < CM) {
    sum = partial[0][lane];
    for (int i = 1; i < kSlices; ++i) sum += partial[i][lane];
    atomicAdd(acc + static_cast<size_t>(blockIdx.x) * CM + cm, sum);
  }
}

template <typename T>
__global__ void __launch_bounds__(256)
    dw_round_kernel(const float* __restrict__ acc, T* __restrict__ out, int n) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i < n) out[i] = Elem<T>::from_float(acc[i]);
}

// Launches the 3x3 strip kernel with V channels per lane and a TH x TW block
// of outputs per lane.  A lane loads (TH + 2)(TW + 2) input vectors for
// TH * TW outputs (stride 1), so larger blocks cut the L1 traffic, but fewer
// lanes remain and, with TW = 2, a wave's loads spread over twice as many
// cache lines.  Measured best on MI355X at batch 32 / 128:
//   stride 1: TW = 2 once a pixel's channel vectors fill a 128-byte line,
//             TH = 4 for images of 28 rows and more, else 8 (4 with V = 8);
//   stride 2: TW = 1, TH = 2 for outputs of 56 rows and more, else 8 (4).
// The tall-strip kernel for the shapes it is built for: fp32, 32 / 64 / 128
// channels, strips of 14 x 4 outputs per lane at stride 1 and 7 x 1 at stride
// 2, enough waves to cover the GPU (smaller launches keep the short strips,
// whose many lanes hide latency better).  Returns false when it does not take
// the launch.
template <typename T, bool FLIP>
bool launch_dw_tall(const T* input, const T* filter, T* output,
                    const snn_hip_depthwise_params& p, hipStream_t stream) {
  constexpr int kV = 16 / sizeof(T);  // channels per lane
  constexpr bool kHalf = sizeof(T) == 2;
  if (p.channels % kV != 0) return false;
  const int cv = p.channels / kV;
  if (cv != 4 && cv != 8 && cv != 16 && cv != 32) return false;
  if (cv == 4 && !kHalf) return false;   // fp32: 32 / 64 / 128 channels
  if (cv == 32 && kHalf) return false;   // half: 32 / 64 / 128 channels
  if (p.pad_rows > 2 || p.pad_cols > 2) return false;
  const int stride = p.stride_rows;
  // Half precision at stride 1 stays on the short strips: measured at batch
  // 128, 112x112x32 runs 44.8 us there against 61 us here (14 x 2 per lane;
  // 57 us at 7 x 4) and 56x56x128 43.6 against 50 us, while the stride-2
  // layer gains (112x112x64: 47.2 -> 44.0 us, 0.73 of the HBM peak).
  if (kHalf && stride == 1 && SNN_TUNING_ENV("SNN_HIP_DW_TALL") == nullptr)
    return false;
  // half keeps eight channels per lane: half the columns for the same bytes
  int th = stride == 1 ? 14 : 7, tw = stride == 1 ? (kHalf ? 2 : 4) : 1;
  // Developer overrides for tuning runs: SNN_HIP_DW_TALL=<th>x<tw> among the
  // shapes instantiated below.
  if (const char* tune = SNN_TUNING_ENV("SNN_HIP_DW_TALL")) {
    int a = 0, b = 0;
    if (sscanf(tune, "%dx%d", &a, &b) == 2) {
      th = a;
      tw = b;
    }
  }
  if (p.out_rows < th) return false;
  const int wpx = (64 / cv) * tw;
  const int n_wcols = ceil_div(p.out_cols, wpx);
  const int n_strips = ceil_div(p.out_rows, th);
  const size_t waves = static_cast<size_t>(p.batch) * n_strips * n_wcols;
  // ragged last wave column: at most a fifth of the lanes idle overall
  if (static_cast<size_t>(n_wcols) * wpx * 4 > static_cast<size_t>(p.out_cols) * 5)
    return false;
  if (waves < 768 || waves > 0x3FFFFFFFu) return false;
  const unsigned n_waves = static_cast<unsigned>(waves);
  const dim3 grid(ceil_div(n_waves, 4u));
#define SNN_DW_TALL(STRIDE, TH, TW, CV)                                         \
  hipLaunchKernelGGL((dw_forward_3x3_tall_kernel<T, STRIDE, TH, TW, CV, FLIP>), \
                     grid, dim3(256), 0, stream, input, filter, output, p,      \
                     n_strips, n_wcols, n_waves)
#define SNN_DW_TALL_CV(STRIDE, TH, TW)                                \
  do {                                                                \
    if constexpr (kHalf) {                                            \
      if (cv == 4) SNN_DW_TALL(STRIDE, TH, TW, 4);                    \
      else if (cv == 8) SNN_DW_TALL(STRIDE, TH, TW, 8);               \
      else SNN_DW_TALL(STRIDE, TH, TW, 16);                           \
    } else {                                                          \
      if (cv == 8) SNN_DW_TALL(STRIDE, TH, TW, 8);                    \
      else if (cv == 16) SNN_DW_TALL(STRIDE, TH, TW, 16);             \
      else SNN_DW_TALL(STRIDE, TH, TW, 32);                           \
    }                                                                 \
  } while (0)
  if (stride == 1) {
    if constexpr (kHalf) {
#ifdef SNN_HIP_TUNING
      if (th == 14 && tw == 2) SNN_DW_TALL_CV(1, 14, 2);
      else if (th == 7 && tw == 4) SNN_DW_TALL_CV(1, 7, 4);
      else if (th == 7 && tw == 2) SNN_DW_TALL_CV(1, 7, 2);
      else if (th == 14 && tw == 1) SNN_DW_TALL_CV(1, 14, 1);
      else
#endif
        return false;
    } else {
      if (th == 14 && tw == 4) SNN_DW_TALL_CV(1, 14, 4);
#ifdef SNN_HIP_TUNING
      else if (th == 14 && tw == 2) SNN_DW_TALL_CV(1, 14, 2);
      else if (th == 7 && tw == 4) SNN_DW_TALL_CV(1, 7, 4);
#endif
      else return false;
    }
  } else {
    if (th == 7 && tw == 1) SNN_DW_TALL_CV(2, 7, 1);
#ifdef SNN_HIP_TUNING
    else if (th == 4 && tw == 1) SNN_DW_TALL_CV(2, 4, 1);
    else if (th == 14 && tw == 1) SNN_DW_TALL_CV(2, 14, 1);
#endif
    else return false;
  }
#undef SNN_DW_TALL_CV
#undef SNN_DW_TALL
  return true;
}

template <typename T, int V, bool FLIP>
void launch_dw_strip(const T* input, const T* filter, T* output,
                     const snn_hip_depthwise_params& p, hipStream_t stream) {
  constexpr int kBlock = 256;
  if constexpr (V * sizeof(T) == 16) {
    if (SNN_TUNING_ENV("SNN_HIP_DW_TALL_OFF") == nullptr &&
        launch_dw_tall<T, FLIP>(input, filter, output, p, stream))
      return;
  }
  const int cv = p.channels / V;
  const int th_max = V == 8 ? 4 : 8;  // 8 rows x 8 channels: ~250 registers
  int th, tw;
  if (p.stride_rows == 1) {
    tw = cv * 16 >= 128 ? 2 : 1;
    // (up to eight rows: two strips of four keep twice the lanes in flight,
    // 7x7x1024 at batch 32 5.7 -> 4.8 us)
    th = (p.out_rows >= 28 || p.out_rows <= 8) ? 4 : th_max;
  } else {
    tw = 1;
    th = p.out_rows >= 56 ? 2 : th_max;
  }
  // Developer overrides for tuning runs: SNN_HIP_DW_TH=<1|2|4|8>,
  // SNN_HIP_DW_TW=<1|2>.
  static const char* tune_th = SNN_TUNING_ENV("SNN_HIP_DW_TH");
  static const char* tune_tw = SNN_TUNING_ENV("SNN_HIP_DW_TW");
  if (tune_th != nullptr && tune_th[0] != 0) th = atoi(tune_th);
  if (tune_tw != nullptr && tune_tw[0] != 0) tw = atoi(tune_tw);
  tw = tw >= 2 ? 2 : 1;
  th = th >= 8 ? 8 : th >= 4 ? 4 : th >= 2 ? 2 : 1;
  if (th > th_max) th = th_max;
  const int n_col_blocks = ceil_div(p.out_cols, tw);
  const int n_strips = ceil_div(p.out_rows, th);
  const unsigned n_items = static_cast<unsigned>(
      static_cast<size_t>(p.batch) * n_col_blocks * cv * n_strips);
  const dim3 grid(ceil_div(n_items, static_cast<unsigned>(kBlock)));
#define SNN_DW_STRIP(STRIDE, TH, TW)                                            \
  hipLaunchKernelGGL((dw_forward_3x3_strip_kernel<T, STRIDE, TH, TW, FLIP, V>), \
                     grid, dim3(kBlock), 0, stream, input, filter, output, p,   \
                     n_strips, n_col_blocks, n_items)
#define SNN_DW_STRIP_TH(STRIDE, TW)                      \
  do {                                                   \
    if (th == 8) {                                       \
      if constexpr (V != 8) SNN_DW_STRIP(STRIDE, 8, TW); \
    } else if (th == 4) {                                \
      SNN_DW_STRIP(STRIDE, 4, TW);                       \
    } else if (th == 2) {                                \
      SNN_DW_STRIP(STRIDE, 2, TW);                       \
    } else {                                             \
      SNN_DW_STRIP(STRIDE, 1, TW);                       \
    }                                                    \
  } while (0)
  if (p.stride_rows == 1) {
    if (tw == 2) SNN_DW_STRIP_TH(1, 2);
    else SNN_DW_STRIP_TH(1, 1);
  } else {
    if (tw == 2) SNN_DW_STRIP_TH(2, 2);
    else SNN_DW_STRIP_TH(2, 1);
  }
#undef SNN_DW_STRIP_TH
#undef SNN_DW_STRIP
}

}  // namespace

// Device memory for the entry point that allocates nothing
// (snn_hip_depthwise_conv2d_filter_backprop_noalloc_f32): the work-groups'
// partial filters.  The strip kernel runs at most 1024 / grid_y + 1 groups
// along x, each writing 9 * C floats with C <= 128 * grid_y, so 2048 * 1152
// floats (9 MiB) hold the partial filters of every shape that kernel takes
// with room to spare.  Every
// device the library runs on holds its own copy until the process ends.
constexpr size_t kDwScratchElems = size_t{2048} * 1152;
static __device__ __align__(256) float scratch[kDwScratchElems];

namespace {

// The address of `scratch` on the current device, looked up once per device.
// In host code the array's name is only a handle for hipGetSymbolAddress;
// kernels and copies must be given the pointer this returns.
int dw_scratch_on_current_device(float** out) {
  constexpr int kMaxDevices = 64;
  static std::mutex mutex;
  static float* address[kMaxDevices] = {};
  int device = 0;
  SNN_HIP_TRY(hipGetDevice(&device));
  if (device < 0 || device >= kMaxDevices)
    return report_error(SNN_HIP_INVALID_PARAMETER,
                        "device ordinal beyond the per-device scratch table");
  std::lock_guard<std::mutex> lock(mutex);
  if (address[device] == nullptr) {
    void* p = nullptr;
    SNN_HIP_TRY(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    address[device] = static_cast<float*>(p);
  }
  *out = address[device];
  return SNN_HIP_OK;
}

}  // namespace

// Picks the strip height (4 or 8 output rows, whichever wastes fewer rows of
// the last row block; 8 on a tie) and deals the strips to the work-groups.
// The work-groups add their sums into the zero-filled dF with float atomics
// while those stay few; otherwise their partial filters go to `static_scratch`
// when the caller brings it (kDwScratchElems floats), else to a stream-ordered
// temporary, and a second kernel adds them up (also the fallback when the
// allocation fails).
template <typename T>
static int launch_dw_filbk_strip(const T* x, const T* dy, float* dw,
                                 const snn_hip_depthwise_params& p, int cvw,
                                 int grid_y, hipStream_t stream,
                                 float* static_scratch) {
  const int n_pl = kDwFilbkThreads / cvw;
  const int th =
      ceil_div(p.out_rows, 8) * 8 <= ceil_div(p.out_rows, 4) * 4 ? 8 : 4;
  constexpr int tw = 2;
  const int n_rb = ceil_div(p.out_rows, th);
  const int n_cb = ceil_div(p.out_cols, tw);
  const int n_strips = p.batch * n_rb * n_cb;
  const int dw_elems = 9 * p.channels;
  auto plan = [&](int target_groups, int* spg) {
    *spg = max(n_pl, ceil_div(n_strips, max(1, target_groups / grid_y)));
    *spg = ceil_div(*spg, n_pl) * n_pl;
    return ceil_div(n_strips, *spg);
  };
  const size_t in_bytes = static_cast<size_t>(p.batch) * p.in_rows *
                          p.in_cols * p.channels * sizeof(T);
  // Large inputs: about 448 work-groups, every lane two or more strips (more,
  // shorter work-groups lose to their own start and end).  Small ones: up to
  // 1024, for the sake of parallelism.
  constexpr size_t kLargeInputBytes = size_t{32} << 20;
  // Above this many float atomics into dF the partial filters and a second
  // kernel are cheaper (measured: about 45 atomics per nanosecond).
  constexpr size_t kMaxAtomics = size_t{1} << 18;
  int spg = 0;
  const int grid_x =
      plan(in_bytes >= kLargeInputBytes ? 448 : 1024, &spg);
  const size_t part_elems = static_cast<size_t>(grid_x) * dw_elems;
  float* part = nullptr;
  bool temporary = false;
  if (part_elems > kMaxAtomics) {
    if (static_scratch != nullptr) {
      if (part_elems > kDwScratchElems)
        return report_error(
            SNN_HIP_INVALID_PARAMETER,
            "depthwise filter backprop without allocation: the partial "
            "filters need " + std::to_string(part_elems * sizeof(float)) +
            " bytes, the library's scratch array holds " +
            std::to_string(kDwScratchElems * sizeof(float)));
      part = static_scratch;
    } else if (temp_malloc_async(reinterpret_cast<void**>(&part),
                              part_elems * sizeof(float),
                              stream) == hipSuccess) {
      temporary = true;
    } else {
      (void)hipGetLastError();
      part = nullptr;
    }
  }
  if (part == nullptr) {
    hipLaunchKernelGGL(dw_zero_kernel, dim3(ceil_div(dw_elems, 256)),
                       dim3(256), 0, stream, dw, dw_elems);
  }
  const dim3 grid(static_cast<unsigned>(grid_x),
                  static_cast<unsigned>(grid_y));
  auto launch = [&](auto kernel) {
    hipLaunchKernelGGL(kernel, grid, dim3(kDwFilbkThreads), 0, stream, x, dy,
                       dw, part, p, cvw, spg, n_strips, n_rb, n_cb);
  };
  // Loads two output rows ahead of the arithmetic at stride 1, one at stride 2
  // (measured at batch 32: 112x112x32 30.1 / 27.5 / 26.5 / 26.4 us for 0 / 1 /
  // 2 / 3 rows, 112x112x64 stride 2 32.6 / 30.1 / 31.1 / 32.6 us).
  if (p.stride_rows == 1) {
    if (th == 8)
      launch((dw_filter_backprop_3x3_strip_kernel<1, 8, tw, 2, T>));
    else
      launch((dw_filter_backprop_3x3_strip_kernel<1, 4, tw, 1, T>));
  } else {
    if (th == 8)
      launch((dw_filter_backprop_3x3_strip_kernel<2, 8, tw, 1, T>));
    else
      launch((dw_filter_backprop_3x3_strip_kernel<2, 4, tw, 1, T>));
  }
  if (part != nullptr) {
    const int n_vec = dw_elems / 4;
    hipLaunchKernelGGL(
        dw_filbk_reduce_kernel,
        dim3(static_cast<unsigned>(ceil_div(n_vec, 64)),
             static_cast<unsigned>(
                 ceil_div(grid_x, 4 * kDwFilbkReduceLoads))),
        dim3(256), 0, stream, reinterpret_cast<const float4*>(part), dw, n_vec,
        grid_x);
    if (temporary) temp_free_async(part, stream);
  }
  return SNN_HIP_OK;
}

template <typename T>
int launch_depthwise(int direction, const T* input, const T* filter, T* output,
                     const snn_hip_depthwise_params& p, hipStream_t stream,
                     float* static_scratch) {
  KernelTimer timer(stream);
  constexpr int kBlock = 256;
  const size_t CM = static_cast<size_t>(p.channels) * p.channel_multiplier;
  if (direction == SNN_HIP_FORWARD) {
    const size_t n_out = static_cast<size_t>(p.batch) * p.out_rows * p.out_cols * CM;
    const bool is3x3 = p.window_rows == 3 && p.window_cols == 3 &&
                       p.stride_rows == p.stride_cols &&
                       (p.stride_rows == 1 || p.stride_rows == 2);
    const bool small = n_out * sizeof(T) < 0x7FFFFFF0u &&
                       static_cast<size_t>(p.batch) * p.in_rows * p.in_cols *
                               p.channels * sizeof(T) < 0x7FFFFFF0u;
    if (p.channel_multiplier == 1 && p.channels % 4 == 0 && is3x3 && small) {
      bool wide = false;
      if constexpr (std::is_same<T, _Float16>::value) {
        if (p.channels % 8 == 0) {
          launch_dw_strip<T, 8, false>(input, filter, output, p, stream);
          wide = true;
        }
      }
      if (!wide) launch_dw_strip<T, 4, false>(input, filter, output, p, stream);
    } else if (p.channel_multiplier == 1 && p.channels % 4 == 0) {
      const size_t n_vec = n_out / 4;
      hipLaunchKernelGGL(dw_forward_vec4_kernel<T>,
                         dim3(static_cast<unsigned>(ceil_div(n_vec, size_t{kBlock}))),
                         dim3(kBlock), 0, stream, input, filter, output, p,
                         n_vec);
    } else {
      hipLaunchKernelGGL(dw_forward_scalar_kernel<T>,
                         dim3(static_cast<unsigned>(ceil_div(n_out, size_t{kBlock}))),
                         dim3(kBlock), 0, stream, input, filter, output, p,
                         n_out);
    }
  } else if (direction == SNN_HIP_INPUT_BACKPROP) {
    const size_t n_out =
        static_cast<size_t>(p.batch) * p.in_rows * p.in_cols * p.channels;
    const bool vec_ok =
        p.channel_multiplier == 1 && p.channels % 4 == 0 &&
        n_out * sizeof(T) < 0x7FFFFFF0u &&
        static_cast<size_t>(p.batch) * p.out_rows * p.out_cols * p.channels *
                sizeof(T) < 0x7FFFFFF0u;
    if (vec_ok && p.window_rows == 3 && p.window_cols == 3 &&
        p.stride_rows == 1 && p.stride_cols == 1 && p.pad_rows <= 2 &&
        p.pad_cols <= 2) {
      // stride 1: the forward strip kernel on dY with the taps reversed
      snn_hip_depthwise_params q = p;
      q.in_rows = p.out_rows;  q.in_cols = p.out_cols;
      q.out_rows = p.in_rows;  q.out_cols = p.in_cols;
      q.pad_rows = 2 - p.pad_rows;
      q.pad_cols = 2 - p.pad_cols;
      bool wide = false;
      if constexpr (std::is_same<T, _Float16>::value) {
        if (q.channels % 8 == 0) {
          launch_dw_strip<T, 8, true>(input, filter, output, q, stream);
          wide = true;
        }
      }
      if (!wide) launch_dw_strip<T, 4, true>(input, filter, output, q, stream);
    } else if (vec_ok && p.window_rows == 3 && p.window_cols == 3 &&
               p.stride_rows == 2 && p.stride_cols == 2 && p.pad_rows <= 2 &&
               p.pad_cols <= 2 && SNN_TUNING_ENV("SNN_HIP_DW_INBK_GATHER") == nullptr) {
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
        hipLaunchKernelGGL((dw_input_backprop_3x3_s2_kernel<T, 4>), grid,
                           dim3(kBlock), 0, stream, input, filter, output, p,
                           n_bcols, n_strips, n_items);
      else
        hipLaunchKernelGGL((dw_input_backprop_3x3_s2_kernel<T, 2>), grid,
                           dim3(kBlock), 0, stream, input, filter, output, p,
                           n_bcols, n_strips, n_items);
    } else if (vec_ok) {
      const unsigned n_vec = static_cast<unsigned>(n_out / 4);
      hipLaunchKernelGGL(dw_input_backprop_vec4_kernel<T>,
                         dim3(ceil_div(n_vec, static_cast<unsigned>(kBlock))),
                         dim3(kBlock), 0, stream, input, filter, output, p,
                         n_vec);
    } else
    hipLaunchKernelGGL(dw_input_backprop_kernel<T>,
                       dim3(static_cast<unsigned>(ceil_div(n_out, size_t{kBlock}))),
                       dim3(kBlock), 0, stream, input, filter, output, p,
                       n_out);
  } else {
    const size_t n_pix_sz =
        static_cast<size_t>(p.batch) * p.out_rows * p.out_cols;
    bool done = false;
    if constexpr (std::is_same<T, _Float16>::value) {
      // binary16, 3x3, stride 1 or 2: the fp32 strip kernel reading binary16,
      // its sums in an fp32 temporary of the filter's size that one more pass
      // rounds (the general kernel below took 1.07 ms where this takes about
      // what fp32 does: 112x112x32 at batch 128)
      if (p.channel_multiplier == 1 && p.channels % 4 == 0 &&
          p.window_rows == 3 && p.window_cols == 3 &&
          p.stride_rows == p.stride_cols &&
          (p.stride_rows == 1 || p.stride_rows == 2) &&
          n_pix_sz * p.channels * sizeof(T) < 0x7FFFFFF0u &&
          static_cast<size_t>(p.batch) * p.in_rows * p.in_cols * p.channels *
                  sizeof(T) < 0x7FFFFFF0u &&
          n_pix_sz * p.channels >= (size_t{1} << 18)) {
        const int cv = p.channels / 4;
        int cvw = 1;
        while (cvw * 2 <= cv && cvw < 32) cvw *= 2;  // >= 8 pixel lanes
        const int grid_y = ceil_div(cv, cvw);
        const int dw_elems = 9 * p.channels;
        void* acc = nullptr;
        if (temp_malloc_async(&acc, dw_elems * sizeof(float), stream) !=
            hipSuccess)
          return SNN_HIP_ALLOCATION_PROBLEM;
        const int status = launch_dw_filbk_strip<T>(
            input, filter, static_cast<float*>(acc), p, cvw, grid_y, stream,
            nullptr);
        if (status == SNN_HIP_OK)
          hipLaunchKernelGGL(dw_round_kernel<T>, dim3(ceil_div(dw_elems, 256)),
                             dim3(256), 0, stream,
                             static_cast<const float*>(acc), output, dw_elems);
        const hipError_t err = hipGetLastError();
        temp_free_async(acc, stream);
        if (status != SNN_HIP_OK) return status;
        if (err != hipSuccess)
          return report_hip_error(err, "binary16 depthwise filter backprop");
        return SNN_HIP_OK;
      }
    }
    if constexpr (std::is_same<T, float>::value) {
      if (p.channel_multiplier == 1 && p.channels % 4 == 0 &&
          p.window_rows == 3 && p.window_cols == 3 &&
          n_pix_sz * p.channels * sizeof(T) < 0x7FFFFFF0u &&
          static_cast<size_t>(p.batch) * p.in_rows * p.in_cols * p.channels *
                  sizeof(T) < 0x7FFFFFF0u) {
        const int cv = p.channels / 4;
        int cvw = 1;
        while (cvw * 2 <= cv && cvw < 32) cvw *= 2;  // >= 8 pixel lanes
        const int n_pl = kDwFilbkThreads / cvw;
        const int grid_y = ceil_div(cv, cvw);
        const int n_pix = static_cast<int>(n_pix_sz);
        // about 1024 work-groups (every one ends with cvw * 36 atomics), each
        // at least 8 passes over its pixel lanes
        int ppg = max(n_pl * 8, ceil_div(n_pix, max(1, 1024 / grid_y)));
        ppg = ceil_div(ppg, n_pl) * n_pl;
        const int grid_x = ceil_div(n_pix, ppg);
        const int dw_elems = 9 * p.channels;
        const bool strip_ok =
            p.stride_rows == p.stride_cols &&
            (p.stride_rows == 1 || p.stride_rows == 2) &&
            SNN_TUNING_ENV("SNN_HIP_DW_FILBK_PIXEL") == nullptr;
        if (strip_ok) {
          const int status = launch_dw_filbk_strip<float>(
              input, filter, output, p, cvw, grid_y, stream, static_scratch);
          if (status != SNN_HIP_OK) return status;
        } else {
          hipLaunchKernelGGL(dw_zero_kernel, dim3(ceil_div(dw_elems, 256)),
                             dim3(256), 0, stream, output, dw_elems);
          hipLaunchKernelGGL(dw_filter_backprop_3x3_kernel,
                             dim3(static_cast<unsigned>(grid_x),
                                  static_cast<unsigned>(grid_y)),
                             dim3(kDwFilbkThreads), 0, stream, input, filter,
                             output, p, cvw, ppg);
        }
        done = true;
      }
    }
    if (!done) {
      const int taps = p.window_rows * p.window_cols;
      const int strips = static_cast<int>(ceil_div(CM, size_t{kStrip}));
      // about 2048 work-groups, each slice with at least 16 pixels
      const int chunks =
          n_pix_sz > 0x7FFFFFFFu
              ? 1
              : max(1, min(2048 / (taps * strips),
                           static_cast<int>(n_pix_sz) / (kSlices * 16)));
      if (chunks == 1) {
        // (one work-group per (tap, strip) walks every pixel: no atomics)
        hipLaunchKernelGGL(dw_filter_backprop_kernel<T>,
                           dim3(static_cast<unsigned>(taps),
                                static_cast<unsigned>(strips)),
                           dim3(kStrip * kSlices), 0, stream, input, filter,
                           output, p);
      } else {
        // fp32 accumulation: the result itself, or for binary16 a temporary
        // that one more pass rounds
        const int dw_elems = taps * static_cast<int>(CM);
        float* acc = reinterpret_cast<float*>(output);
        if constexpr (!std::is_same<T, float>::value) {
          void* ptr = nullptr;
          if (temp_malloc_async(&ptr, dw_elems * sizeof(float), stream) !=
              hipSuccess)
            return SNN_HIP_ALLOCATION_PROBLEM;
          acc = static_cast<float*>(ptr);
        }
        const int per_chunk = ceil_div(static_cast<int>(n_pix_sz), chunks);
        hipLaunchKernelGGL(dw_zero_kernel, dim3(ceil_div(dw_elems, 256)),
                           dim3(256), 0, stream, acc, dw_elems);
        hipLaunchKernelGGL(
            dw_filter_backprop_split_kernel<T>,
            dim3(static_cast<unsigned>(taps), static_cast<unsigned>(strips),
                 static_cast<unsigned>(
                     ceil_div(static_cast<int>(n_pix_sz), per_chunk))),
            dim3(kStrip * kSlices), 0, stream, input, filter, acc, p,
            per_chunk);
        if constexpr (!std::is_same<T, float>::value) {
          hipLaunchKernelGGL(dw_round_kernel<T>, dim3(ceil_div(dw_elems, 256)),
                             dim3(256), 0, stream, acc, output, dw_elems);
          const hipError_t err = hipGetLastError();
          temp_free_async(acc, stream);
          if (err != hipSuccess)
            return report_hip_error(err, "depthwise filter backprop");
        }
      }
    }
  }
  SNN_HIP_CHECK_LAUNCH();
  return SNN_HIP_OK;
}

template int launch_depthwise<float>(int, const float*, const float*, float*,
                                     const snn_hip_depthwise_params&,
                                     hipStream_t, float*);
template int launch_depthwise<_Float16>(int, const _Float16*, const _Float16*,
                                        _Float16*,
                                        const snn_hip_depthwise_params&,
                                        hipStream_t, float*);

int launch_depthwise_filter_backprop_noalloc_f32(
    const float* input, const float* dy, float* dw,
    const snn_hip_depthwise_params& p, hipStream_t stream) {
  float* scratch_ptr = nullptr;
  const int status = dw_scratch_on_current_device(&scratch_ptr);
  if (status != SNN_HIP_OK) return status;
  return launch_depthwise<float>(SNN_HIP_FILTER_BACKPROP, input, dy, dw, p,
                                 stream, scratch_ptr);
}

}  // namespace snn
