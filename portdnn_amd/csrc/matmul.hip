// Batched row-major GEMM  C[b] = op(A[b]) * op(B[b]) + beta * C[b]  for gfx950.
// Stand-in for portDNN's MatmulKernel (src/matmul/kernels.h:26-133,
// src/matmul/launch.cc:51-56).
//
// Shapes the matrix-core kernel takes (see launch_matmul_f32) go to it; this
// file holds the general-shape kernel: 64x64 output tile per 256-lane
// work-group, A and B tiles staged in LDS, 4x4 register block per lane, every
// edge bounds-checked so any m, k, n and both transposes are accepted.
#include "snn_kernels.h"

namespace snn {
namespace {

constexpr int kTile = 64;
constexpr int kTileK = 16;

// T = float or _Float16 (products and sums in fp32 either way).
template <bool TransA, bool TransB, typename T = float>
__global__ void __launch_bounds__(256)
    matmul_general_kernel(const T* __restrict__ a, const T* __restrict__ b,
                          T* __restrict__ c, int m, int k, int n, float beta) {
  __shared__ float sa[kTileK][kTile + 4];  // [kk][row]
  __shared__ float sb[kTileK][kTile + 4];  // [kk][col]
  const int batch = blockIdx.z;
  a += static_cast<size_t>(batch) * m * k;
  b += static_cast<size_t>(batch) * k * n;
  c += static_cast<size_t>(batch) * m * n;
  const int row0 = blockIdx.x * kTile;
  const int col0 = blockIdx.y * kTile;
  const int tx = threadIdx.x % 16;  // column group
  const int ty = threadIdx.x / 16;  // row group
  float acc[4][4] = {};
  for (int k0 = 0; k0 < k; k0 += kTileK) {
    for (int e = threadIdx.x; e < kTile * kTileK; e += 256) {
      // A tile element (row r, depth kk)
      int r, kk;
      if (TransA) {  // memory is [k][m]: consecutive lanes walk rows
        r = e % kTile;
        kk = e / kTile;
      } else {  // memory is [m][k]: consecutive lanes walk depth
        kk = e % kTileK;
        r = e / kTileK;
      }
      const int gr = row0 + r, gk = k0 + kk;
      float v = 0.f;
      if (gr < m && gk < k) {
        v = static_cast<float>(TransA ? a[static_cast<size_t>(gk) * m + gr]
                                      : a[static_cast<size_t>(gr) * k + gk]);
      }
      sa[kk][r] = v;
      // B tile element (depth kk2, col cc)
      int cc, kk2;
      if (TransB) {  // memory is [n][k]
        kk2 = e % kTileK;
        cc = e / kTileK;
      } else {  // memory is [k][n]
        cc = e % kTile;
        kk2 = e / kTile;
      }
      const int gc = col0 + cc, gk2 = k0 + kk2;
      float w = 0.f;
      if (gc < n && gk2 < k) {
        w = static_cast<float>(TransB ? b[static_cast<size_t>(gc) * k + gk2]
                                      : b[static_cast<size_t>(gk2) * n + gc]);
      }
      sb[kk2][cc] = w;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < kTileK; ++kk) {
      float av[4], bv[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) av[i] = sa[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) bv[j] = sb[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(av[i], bv[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int gr = row0 + ty * 4 + i;
    if (gr >= m) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int gc = col0 + tx * 4 + j;
      if (gc >= n) continue;
      const size_t o = static_cast<size_t>(gr) * n + gc;
      c[o] = static_cast<T>(
          (beta == 0.f) ? acc[i][j]
                        : fmaf(beta, static_cast<float>(c[o]), acc[i][j]));
    }
  }
}

__global__ void __launch_bounds__(256)
    scale_kernel(float* __restrict__ c, size_t n, float beta) {
  const size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
  if (i < n) c[i] *= beta;
}

// out[r][c] (rows2 x cols2, row-major) = in[r * row_stride + c * col_stride]
// for r < rows and c < cols, else 0: copies a matrix, transposing and / or
// widening it with zeros.
__global__ void __launch_bounds__(256)
    repack_matrix_kernel(const float* __restrict__ in, float* __restrict__ out,
                         int rows, int cols, size_t row_stride,
                         size_t col_stride, int cols2, size_t total) {
  const size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
  if (i >= total) return;
  const size_t r = i / cols2;
  const int c = static_cast<int>(i - r * cols2);
  out[i] = (r < static_cast<size_t>(rows) && c < cols)
               ? in[r * row_stride + c * col_stride]
               : 0.f;
}

void repack_matrix(const float* in, float* out, int rows, int cols,
                   size_t row_stride, size_t col_stride, int rows2, int cols2,
                   hipStream_t stream) {
  const size_t total = static_cast<size_t>(rows2) * cols2;
  hipLaunchKernelGGL(repack_matrix_kernel,
                     dim3(static_cast<unsigned>(ceil_div(total, size_t{256}))),
                     dim3(256), 0, stream, in, out, rows, cols, row_stride,
                     col_stride, cols2, total);
}

// One large product the matrix-core kernel does not take as it stands (A
// transposed, k not a multiple of 32, n not a multiple of 4): the operands
// that do not fit are rewritten into stream-ordered temporaries -- A as m x
// k', B as k' x n', zeros in the new rows and columns -- the kernel runs on
// those, and a widened result is copied back.  The copies move O(mk + kn +
// mn) floats against the O(mkn) of the product.  Returns -1 when it does not
// apply.
int launch_matmul_repacked_f32(const float* lhs, const float* rhs,
                               float* output, int m, int k, int n,
                               bool transpose_lhs, bool transpose_rhs,
                               hipStream_t stream) {
  if (m < 32 || static_cast<double>(m) * k * n < double(1 << 24)) return -1;
  const int k2 = (k + 31) / 32 * 32;
  // (B stored n x k is taken with any n)
  const bool keep_bt = transpose_rhs && k2 == k;
  const int n2 = keep_bt ? n : (n + 3) / 4 * 4;
  const bool new_a = transpose_lhs || k2 != k;
  const bool new_b = !keep_bt && (transpose_rhs || k2 != k || n2 != n);
  const bool new_c = n2 != n;
  if ((reinterpret_cast<uintptr_t>(lhs) | reinterpret_cast<uintptr_t>(rhs) |
       reinterpret_cast<uintptr_t>(output)) & 15u)
    return -1;
  float *a2 = nullptr, *b2 = nullptr, *c2 = nullptr;
  auto release = [&]() {
    if (c2 != nullptr) temp_free_async(c2, stream);
    if (b2 != nullptr) temp_free_async(b2, stream);
    if (a2 != nullptr) temp_free_async(a2, stream);
  };
  auto grab = [&](float** ptr, size_t elems) {
    void* raw = nullptr;
    if (temp_malloc_async(&raw, elems * sizeof(float), stream) != hipSuccess)
      return false;
    *ptr = static_cast<float*>(raw);
    return true;
  };
  if ((new_a && !grab(&a2, static_cast<size_t>(m) * k2)) ||
      (new_b && !grab(&b2, static_cast<size_t>(k2) * n2)) ||
      (new_c && !grab(&c2, static_cast<size_t>(m) * n2))) {
    // (no room for the copies: the general kernel takes the product)
    (void)hipGetLastError();
    release();
    return -1;
  }
  const float* a = new_a ? a2 : lhs;
  const float* b = new_b ? b2 : rhs;
  float* c = new_c ? c2 : output;
  if (!batched_gemm_mfma_supports(m, k2, n2, a, b, c, keep_bt)) {
    release();
    return -1;
  }
  if (new_a)  // A[i][j]: stored m x k, or (transposed) k x m
    repack_matrix(lhs, a2, m, k, transpose_lhs ? 1 : k, transpose_lhs ? m : 1,
                  m, k2, stream);
  if (new_b)  // B[i][j]: stored k x n, or (transposed) n x k
    repack_matrix(rhs, b2, k, n, transpose_rhs ? 1 : n, transpose_rhs ? k : 1,
                  k2, n2, stream);
  const int status = launch_batched_gemm_mfma_f32(a, b, c, 1, m, k2, n2, stream,
                                                  keep_bt, false);
  if (new_c) repack_matrix(c2, output, m, n, n2, 1, m, n, stream);
  const hipError_t err = hipGetLastError();
  release();
  if (status != SNN_HIP_OK) return status;
  if (err != hipSuccess) return report_hip_error(err, "repacked matmul");
  return SNN_HIP_OK;
}

}  // namespace

int launch_matmul_f32(const float* lhs, const float* rhs, float* output,
                      int batches, int m, int k, int n, bool transpose_lhs,
                      bool transpose_rhs, float beta, hipStream_t stream) {
  // Matrix-core path: A not transposed, k a multiple of 32, operands aligned
  // (the implicit-GEMM kernel of the 1x1 convolution; B^T is its K-contiguous
  // filter layout).  beta == 0 overwrites, beta != 0 first scales C in place
  // (unless beta == 1) and then accumulates with float atomics.
  if (!transpose_lhs && m >= 32 &&
      batched_gemm_mfma_supports(m, k, n, lhs, rhs, output, transpose_rhs) &&
      (batches == 1 || (static_cast<size_t>(m) * n) % 4 == 0)) {
    const bool accumulate = beta != 0.f;
    if (accumulate && beta != 1.f) {
      const size_t total = static_cast<size_t>(batches) * m * n;
      hipLaunchKernelGGL(scale_kernel,
                         dim3(static_cast<unsigned>(ceil_div(total, size_t{256}))),
                         dim3(256), 0, stream, output, total, beta);
    }
    return launch_batched_gemm_mfma_f32(lhs, rhs, output, batches, m, k, n,
                                        stream, transpose_rhs, accumulate);
  }
  // A^T B with both operands stored [k x .]: the filter gradient of a 1x1
  // convolution over k pixels with m channels and n features, on its kernel
  // (partial results, if any, in a stream-ordered temporary).
  if (transpose_lhs && !transpose_rhs && batches == 1 && beta == 0.f &&
      ((reinterpret_cast<uintptr_t>(lhs) | reinterpret_cast<uintptr_t>(rhs) |
        reinterpret_cast<uintptr_t>(output)) & 15u) == 0) {
    snn_hip_conv2d_params p = {};
    p.batch = 1;
    p.in_rows = p.out_rows = 1;
    p.in_cols = p.out_cols = k;
    p.window_rows = p.window_cols = 1;
    p.stride_rows = p.stride_cols = 1;
    p.dilation_rows = p.dilation_cols = 1;
    p.groups = 1;
    p.channels = m;
    p.features = n;
    if (conv2d_filter_backprop_direct_f32_supports(p)) {
      const size_t part_floats =
          conv2d_filter_backprop_direct_f32_partial_floats(p);
      void* part = nullptr;
      if (part_floats != 0 &&
          temp_malloc_async(&part, part_floats * sizeof(float), stream) !=
              hipSuccess)
        return SNN_HIP_ALLOCATION_PROBLEM;
      const int status = launch_conv2d_filter_backprop_direct_f32(
          lhs, rhs, output, static_cast<float*>(part), p, stream);
      const hipError_t err = hipGetLastError();
      if (part != nullptr) temp_free_async(part, stream);
      if (status != SNN_HIP_OK) return status;
      SNN_HIP_TRY(err);
      return SNN_HIP_OK;
    }
  }
  if (batches == 1 && beta == 0.f) {
    const int repacked = launch_matmul_repacked_f32(
        lhs, rhs, output, m, k, n, transpose_lhs, transpose_rhs, stream);
    if (repacked >= 0) return repacked;
  }
  const dim3 grid(static_cast<unsigned>(ceil_div(m, kTile)),
                  static_cast<unsigned>(ceil_div(n, kTile)),
                  static_cast<unsigned>(batches));
  const dim3 block(256);
  if (transpose_lhs) {
    if (transpose_rhs)
      hipLaunchKernelGGL((matmul_general_kernel<true, true>), grid, block, 0,
                         stream, lhs, rhs, output, m, k, n, beta);
    else
      hipLaunchKernelGGL((matmul_general_kernel<true, false>), grid, block, 0,
                         stream, lhs, rhs, output, m, k, n, beta);
  } else {
    if (transpose_rhs)
      hipLaunchKernelGGL((matmul_general_kernel<false, true>), grid, block, 0,
                         stream, lhs, rhs, output, m, k, n, beta);
    else
      hipLaunchKernelGGL((matmul_general_kernel<false, false>), grid, block, 0,
                         stream, lhs, rhs, output, m, k, n, beta);
  }
  SNN_HIP_CHECK_LAUNCH();
  return SNN_HIP_OK;
}

int launch_matmul_f16(const _Float16* lhs, const _Float16* rhs,
                      _Float16* output, int batches, int m, int k, int n,
                      bool transpose_lhs, bool transpose_rhs, float beta,
                      hipStream_t stream) {
  // Matrix-core path: one problem, A not transposed, beta == 0 and operands
  // the half-precision 1x1 convolution kernels take.  A [m x k] * B [k x n]
  // is the forward 1x1 convolution of m pixels with k channels and n
  // features (B is its HWCF filter); A * B^T with B stored [n x k] is the
  // input gradient of the 1x1 convolution with n channels and k features.
  const bool aligned =
      ((reinterpret_cast<uintptr_t>(lhs) | reinterpret_cast<uintptr_t>(rhs) |
        reinterpret_cast<uintptr_t>(output)) & 15u) == 0;
  if (!transpose_lhs && batches == 1 && beta == 0.f && aligned && m >= 32) {
    snn_hip_conv2d_params p = {};
    p.batch = 1;
    p.in_rows = p.out_rows = 1;
    p.in_cols = p.out_cols = m;
    p.window_rows = p.window_cols = 1;
    p.stride_rows = p.stride_cols = 1;
    p.dilation_rows = p.dilation_cols = 1;
    p.groups = 1;
    if (!transpose_rhs) {
      p.channels = k;
      p.features = n;
      if (conv2d_igemm_f16_supports(p))
        return launch_conv2d_igemm_f16(lhs, rhs, output, p, nullptr, 0,
                                       stream);
    } else {
      p.channels = n;
      p.features = k;
      if (conv2d_input_backprop_f16_supports(p))
        return launch_conv2d_input_backprop_f16(lhs, rhs, output, p, nullptr,
                                                0, stream);
    }
  }
  const dim3 grid(static_cast<unsigned>(ceil_div(m, kTile)),
                  static_cast<unsigned>(ceil_div(n, kTile)),
                  static_cast<unsigned>(batches));
  const dim3 block(256);
  if (transpose_lhs) {
    if (transpose_rhs)
      hipLaunchKernelGGL((matmul_general_kernel<true, true, _Float16>), grid,
                         block, 0, stream, lhs, rhs, output, m, k, n, beta);
    else
      hipLaunchKernelGGL((matmul_general_kernel<true, false, _Float16>), grid,
                         block, 0, stream, lhs, rhs, output, m, k, n, beta);
  } else {
    if (transpose_rhs)
      hipLaunchKernelGGL((matmul_general_kernel<false, true, _Float16>), grid,
                         block, 0, stream, lhs, rhs, output, m, k, n, beta);
    else
      hipLaunchKernelGGL((matmul_general_kernel<false, false, _Float16>), grid,
                         block, 0, stream, lhs, rhs, output, m, k, n, beta);
  }
  SNN_HIP_CHECK_LAUNCH();
  return SNN_HIP_OK;
}

}  // namespace snn
