// Element-wise operators: pointwise (relu, tanh, exp, log, floor, sqrt and
// their gradients) and broadcasting binary operators (add, sub, mul, div).
//
// portDNN: src/pointwise/kernels.h:36-246 (operators and the vectorised
// PointwiseOp kernels), src/binaryop/kernels.h:33-250 (operators, the general
// broadcasting kernel and its vector / 2-D broadcast specialisations).
//
// All of these are HBM-bound streams: a lane moves 16 bytes per operand per
// access (float4 or eight halves), a work-group of 256 lanes covers four such
// vectors per lane so that enough loads are in flight, and arithmetic is in
// fp32 for both element types.  The binary operator has three kernels: equal
// shapes (or one scalar operand), an operand that repeats with a period
// dividing the output (bias-like: its shape is the trailing dimensions of the
// output), and the general 4-D index arithmetic of the reference for
// everything else.
#include <algorithm>

#include "snn_kernels.h"

namespace snn {
namespace {

constexpr int kThreads = 256;
constexpr int kUnroll = 4;

template <typename T>
struct Vec16;
template <>
struct Vec16<float> {
  typedef float type __attribute__((ext_vector_type(4)));
  static constexpr int kLanes = 4;
};
template <>
struct Vec16<_Float16> {
  typedef _Float16 type __attribute__((ext_vector_type(8)));
  static constexpr int kLanes = 8;
};

// src/pointwise/kernels.h: Relu :47-49, Tanh :69-71, Exp :91-93, Log :116-118,
// Floor :137-139, Sqrt :152-154.
template <int OP>
__device__ inline float pointwise_fwd(float v) {
  if (OP == SNN_HIP_POINTWISE_RELU) return fmaxf(v, 0.f);
  if (OP == SNN_HIP_POINTWISE_TANH) return tanhf(v);
  if (OP == SNN_HIP_POINTWISE_EXP) return expf(v);
  if (OP == SNN_HIP_POINTWISE_LOG) return logf(v);
  if (OP == SNN_HIP_POINTWISE_FLOOR) return floorf(v);
  return sqrtf(v);
}

// src/pointwise/kernels.h: Relu :53-57, Tanh :75-77, Exp :100-102 (exp(val) +
// err, as written there), Log :122-124, Sqrt :158-160.
template <int OP>
__device__ inline float pointwise_bwd(float v, float e) {
  if (OP == SNN_HIP_POINTWISE_RELU) return v > 0.f ? e : 0.f;
  if (OP == SNN_HIP_POINTWISE_TANH) return (1.f - v * v) * e;
  if (OP == SNN_HIP_POINTWISE_EXP) return expf(v) + e;
  if (OP == SNN_HIP_POINTWISE_LOG) return (1.f / v) * e;
  return (0.5f / v) * e;
}

// src/binaryop/kernels.h:33-59.
template <int OP>
__device__ inline float binary_apply(float a, float b) {
  if (OP == SNN_HIP_BINARY_ADD) return a + b;
  if (OP == SNN_HIP_BINARY_SUB) return a - b;
  if (OP == SNN_HIP_BINARY_MUL) return a * b;
  return a / b;
}

// ---- pointwise -------------------------------------------------------------
// `n_vec` whole vectors, then the tail element by element (last work-group).
template <typename T, int OP, bool GRAD>
__global__ void __launch_bounds__(kThreads)
    pointwise_kernel(const T* in, const T* err, T* out, size_t n_vec,
                     size_t n) {
  typedef typename Vec16<T>::type V;
  constexpr int L = Vec16<T>::kLanes;
  const size_t base =
      static_cast<size_t>(blockIdx.x) * (kThreads * kUnroll) + threadIdx.x;
  V a[kUnroll], e[kUnroll];
#pragma unroll
  for (int u = 0; u < kUnroll; ++u) {
    const size_t i = base + static_cast<size_t>(u) * kThreads;
    if (i < n_vec) {
      a[u] = __builtin_nontemporal_load(reinterpret_cast<const V*>(in) + i);
      if (GRAD)
        e[u] = __builtin_nontemporal_load(reinterpret_cast<const V*>(err) + i);
    }
  }
#pragma unroll
  for (int u = 0; u < kUnroll; ++u) {
    const size_t i = base + static_cast<size_t>(u) * kThreads;
    if (i < n_vec) {
      V r;
#pragma unroll
      for (int k = 0; k < L; ++k) {
        const float v = static_cast<float>(a[u][k]);
        r[k] = static_cast<T>(
            GRAD ? pointwise_bwd<OP>(v, static_cast<float>(e[u][k]))
                 : pointwise_fwd<OP>(v));
      }
      __builtin_nontemporal_store(r, reinterpret_cast<V*>(out) + i);
    }
  }
  if (blockIdx.x == gridDim.x - 1) {
    const size_t i = n_vec * L + threadIdx.x;
    if (i < n) {
      const float v = static_cast<float>(in[i]);
      out[i] = static_cast<T>(
          GRAD ? pointwise_bwd<OP>(v, static_cast<float>(err[i]))
               : pointwise_fwd<OP>(v));
    }
  }
}

// Operands that are not 16-byte aligned: one element per lane.
template <typename T, int OP, bool GRAD>
__global__ void __launch_bounds__(kThreads)
    pointwise_scalar_kernel(const T* in, const T* err, T* out, size_t n) {
  const size_t i = static_cast<size_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (i >= n) return;
  const float v = static_cast<float>(in[i]);
  out[i] = static_cast<T>(GRAD
                              ? pointwise_bwd<OP>(v, static_cast<float>(err[i]))
                              : pointwise_fwd<OP>(v));
}

inline bool aligned16(const void* p) {
  return (reinterpret_cast<uintptr_t>(p) & 15u) == 0;
}

template <typename T, int OP, bool GRAD>
int launch_pointwise_op(const T* in, const T* err, T* out, size_t n,
                        hipStream_t stream) {
  constexpr int L = Vec16<T>::kLanes;
  const bool vec = aligned16(in) && aligned16(out) && (!GRAD || aligned16(err));
  KernelTimer timer(stream);
  if (vec) {
    const size_t n_vec = n / L;
    const size_t groups =
        std::max<size_t>(1, ceil_div(n_vec, size_t{kThreads * kUnroll}));
    hipLaunchKernelGGL((pointwise_kernel<T, OP, GRAD>),
                       dim3(static_cast<unsigned>(groups)), dim3(kThreads), 0,
                       stream, in, err, out, n_vec, n);
  } else {
    hipLaunchKernelGGL((pointwise_scalar_kernel<T, OP, GRAD>),
                       dim3(static_cast<unsigned>(ceil_div(n, size_t{kThreads}))),
                       dim3(kThreads), 0, stream, in, err, out, n);
  }
  const hipError_t e = hipGetLastError();
  return e == hipSuccess ? SNN_HIP_OK : report_hip_error(e, "pointwise_kernel");
}

template <typename T, bool GRAD>
int dispatch_pointwise(int op, const T* in, const T* err, T* out, size_t n,
                       hipStream_t stream) {
  switch (op) {
    case SNN_HIP_POINTWISE_RELU:
      return launch_pointwise_op<T, SNN_HIP_POINTWISE_RELU, GRAD>(in, err, out,
                                                                  n, stream);
    case SNN_HIP_POINTWISE_TANH:
      return launch_pointwise_op<T, SNN_HIP_POINTWISE_TANH, GRAD>(in, err, out,
                                                                  n, stream);
    case SNN_HIP_POINTWISE_EXP:
      return launch_pointwise_op<T, SNN_HIP_POINTWISE_EXP, GRAD>(in, err, out,
                                                                 n, stream);
    case SNN_HIP_POINTWISE_LOG:
      return launch_pointwise_op<T, SNN_HIP_POINTWISE_LOG, GRAD>(in, err, out,
                                                                 n, stream);
    case SNN_HIP_POINTWISE_FLOOR:
      if (GRAD) return SNN_HIP_INVALID_PARAMETER;  // Floor has no gradient
      return launch_pointwise_op<T, SNN_HIP_POINTWISE_FLOOR, false>(
          in, err, out, n, stream);
    case SNN_HIP_POINTWISE_SQRT:
      return launch_pointwise_op<T, SNN_HIP_POINTWISE_SQRT, GRAD>(in, err, out,
                                                                  n, stream);
    default:
      return SNN_HIP_INVALID_PARAMETER;
  }
}

// ---- binaryop --------------------------------------------------------------
// Operand index modes of the vector kernel.
constexpr int kFull = 0;    // same element as the output
constexpr int kScalar = 1;  // one element
constexpr int kPeriod = 2;  // repeats every `period` elements (period % L == 0)

template <typename T, int OP, int LHS_MODE, int RHS_MODE>
__global__ void __launch_bounds__(kThreads)
    binary_vec_kernel(const T* lhs, const T* rhs, T* out, size_t n_vec,
                      size_t n, unsigned period_vecs) {
  typedef typename Vec16<T>::type V;
  constexpr int L = Vec16<T>::kLanes;
  const size_t base =
      static_cast<size_t>(blockIdx.x) * (kThreads * kUnroll) + threadIdx.x;
  auto load = [&](const T* p, int mode, size_t i) {
    V v;
    if (mode == kFull) {
      v = __builtin_nontemporal_load(reinterpret_cast<const V*>(p) + i);
    } else if (mode == kPeriod) {
      v = reinterpret_cast<const V*>(p)[i % period_vecs];
    } else {
      const T s = p[0];
#pragma unroll
      for (int k = 0; k < L; ++k) v[k] = s;
    }
    return v;
  };
  V a[kUnroll], b[kUnroll];
#pragma unroll
  for (int u = 0; u < kUnroll; ++u) {
    const size_t i = base + static_cast<size_t>(u) * kThreads;
    if (i < n_vec) {
      a[u] = load(lhs, LHS_MODE, i);
      b[u] = load(rhs, RHS_MODE, i);
    }
  }
#pragma unroll
  for (int u = 0; u < kUnroll; ++u) {
    const size_t i = base + static_cast<size_t>(u) * kThreads;
    if (i < n_vec) {
      V r;
#pragma unroll
      for (int k = 0; k < L; ++k)
        r[k] = static_cast<T>(binary_apply<OP>(static_cast<float>(a[u][k]),
                                               static_cast<float>(b[u][k])));
      __builtin_nontemporal_store(r, reinterpret_cast<V*>(out) + i);
    }
  }
  // Tail (kFull / kScalar operands only; a periodic operand divides n).
  if (blockIdx.x == gridDim.x - 1) {
    const size_t i = n_vec * L + threadIdx.x;
    if (i < n) {
      const float x = static_cast<float>(lhs[LHS_MODE == kScalar ? 0 : i]);
      const float y = static_cast<float>(rhs[RHS_MODE == kScalar ? 0 : i]);
      out[i] = static_cast<T>(binary_apply<OP>(x, y));
    }
  }
}

struct Dims4 {
  int d[4];
};

// src/binaryop/kernels.h:86-124: one lane per output element; an operand
// index advances along a dimension only where that operand is not broadcast.
template <typename T, int OP>
__global__ void __launch_bounds__(kThreads)
    binary_general_kernel(const T* lhs, const T* rhs, T* out, Dims4 l,
                          Dims4 r, Dims4 o, size_t n) {
  const size_t idx = static_cast<size_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (idx >= n) return;
  size_t rem = idx, li = 0, ri = 0, ls = 1, rs = 1;
#pragma unroll
  for (int d = 3; d >= 0; --d) {
    const size_t c = d > 0 ? rem % o.d[d] : rem;
    if (c < static_cast<size_t>(l.d[d])) li += c * ls;
    if (c < static_cast<size_t>(r.d[d])) ri += c * rs;
    ls *= l.d[d];
    rs *= r.d[d];
    if (d > 0) rem /= o.d[d];
  }
  out[idx] = static_cast<T>(binary_apply<OP>(static_cast<float>(lhs[li]),
                                             static_cast<float>(rhs[ri])));
}

// How an operand with right-aligned dims `d` maps onto output dims `o`:
// kFull, kScalar, kPeriod (returns the period through *period) or -1.
int classify(const Dims4& d, const Dims4& o, size_t* period) {
  size_t size = 1, out_size = 1;
  for (int i = 0; i < 4; ++i) {
    size *= d.d[i];
    out_size *= o.d[i];
  }
  if (size == out_size) return kFull;
  if (size == 1) return kScalar;
  // Trailing dimensions equal to the output's, leading ones all 1.
  int i = 3;
  size_t trailing = 1;
  while (i >= 0 && d.d[i] == o.d[i]) trailing *= d.d[i--];
  for (; i >= 0; --i)
    if (d.d[i] != 1) return -1;
  *period = trailing;
  return kPeriod;
}

template <typename T, int OP>
int launch_binary_op(const T* lhs, const T* rhs, T* out, const Dims4& l,
                     const Dims4& r, const Dims4& o, hipStream_t stream) {
  constexpr int L = Vec16<T>::kLanes;
  size_t n = 1;
  for (int i = 0; i < 4; ++i) n *= o.d[i];
  size_t lp = 0, rp = 0;
  const int lm = classify(l, o, &lp), rm = classify(r, o, &rp);
  const bool aligned = aligned16(lhs) && aligned16(rhs) && aligned16(out);
  const bool periodic_ok = (lm != kPeriod || lp % L == 0) &&
                           (rm != kPeriod || rp % L == 0) &&
                           !(lm == kPeriod && rm == kPeriod);
  if (aligned && lm >= 0 && rm >= 0 && periodic_ok) {
    const size_t n_vec = n / L;
    const unsigned groups = static_cast<unsigned>(
        std::max<size_t>(1, ceil_div(n_vec, size_t{kThreads * kUnroll})));
    const unsigned period =
        static_cast<unsigned>((lm == kPeriod ? lp : rp) / L);
#define SNN_BINARY_CASE(LM, RM)                                              \
  if (lm == LM && rm == RM) {                                                \
    hipLaunchKernelGGL((binary_vec_kernel<T, OP, LM, RM>), dim3(groups),     \
                       dim3(kThreads), 0, stream, lhs, rhs, out, n_vec, n,   \
                       period);                                              \
  }
    SNN_BINARY_CASE(kFull, kFull)
    SNN_BINARY_CASE(kFull, kScalar)
    SNN_BINARY_CASE(kScalar, kFull)
    SNN_BINARY_CASE(kScalar, kScalar)
    SNN_BINARY_CASE(kFull, kPeriod)
    SNN_BINARY_CASE(kPeriod, kFull)
    SNN_BINARY_CASE(kScalar, kPeriod)
    SNN_BINARY_CASE(kPeriod, kScalar)
#undef SNN_BINARY_CASE
  } else {
    hipLaunchKernelGGL((binary_general_kernel<T, OP>),
                       dim3(static_cast<unsigned>(ceil_div(n, size_t{kThreads}))),
                       dim3(kThreads), 0, stream, lhs, rhs, out, l, r, o, n);
  }
  const hipError_t e = hipGetLastError();
  return e == hipSuccess ? SNN_HIP_OK : report_hip_error(e, "binary kernel");
}

template <typename T>
int launch_binaryop_t(int op, const T* lhs, const T* rhs, T* out,
                      const int* lhs_dims, int n_lhs, const int* rhs_dims,
                      int n_rhs, hipStream_t stream) {
  // include/portdnn/internal/binaryop/launch.h:40-62 and :78-101: at most
  // four dimensions each, right-aligned, sizes positive, a dimension of 1
  // broadcasts.
  if (n_lhs < 0 || n_rhs < 0 || n_lhs > 4 || n_rhs > 4)
    return SNN_HIP_INVALID_PARAMETER;
  Dims4 l = {{1, 1, 1, 1}}, r = {{1, 1, 1, 1}}, o;
  for (int i = 0; i < n_lhs; ++i) l.d[4 - n_lhs + i] = lhs_dims[i];
  for (int i = 0; i < n_rhs; ++i) r.d[4 - n_rhs + i] = rhs_dims[i];
  size_t n = 1;
  for (int i = 0; i < 4; ++i) {
    if (l.d[i] < 1 || r.d[i] < 1) return SNN_HIP_INVALID_PARAMETER;
    if (l.d[i] != r.d[i] && l.d[i] != 1 && r.d[i] != 1)
      return SNN_HIP_INVALID_PARAMETER;
    o.d[i] = l.d[i] > r.d[i] ? l.d[i] : r.d[i];
    n *= o.d[i];
  }
  if (n > 0x7FFFFFFFu) return SNN_HIP_INDEX_EXCEEDED;
  switch (op) {
    case SNN_HIP_BINARY_ADD:
      return launch_binary_op<T, SNN_HIP_BINARY_ADD>(lhs, rhs, out, l, r, o,
                                                     stream);
    case SNN_HIP_BINARY_SUB:
      return launch_binary_op<T, SNN_HIP_BINARY_SUB>(lhs, rhs, out, l, r, o,
                                                     stream);
    case SNN_HIP_BINARY_MUL:
      return launch_binary_op<T, SNN_HIP_BINARY_MUL>(lhs, rhs, out, l, r, o,
                                                     stream);
    case SNN_HIP_BINARY_DIV:
      return launch_binary_op<T, SNN_HIP_BINARY_DIV>(lhs, rhs, out, l, r, o,
                                                     stream);
    default:
      return SNN_HIP_INVALID_PARAMETER;
  }
}

// data = act(data + bias[feature]) in place; VEC lanes of one vector share a
// pixel (features % 4 == 0) or the kernel runs element by element.
template <bool VEC>
__global__ void __launch_bounds__(kThreads)
    bias_act_kernel(float* data, const float* __restrict__ bias,
                    unsigned features, size_t n_items, int relu) {
  typedef Vec16<float>::type V;
  const size_t i = static_cast<size_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (i >= n_items) return;
  if (VEC) {
    V v = reinterpret_cast<V*>(data)[i];
    if (bias != nullptr) {
      const V b = *reinterpret_cast<const V*>(
          bias + static_cast<unsigned>((i * 4) % features));
      v += b;
    }
    if (relu) {
#pragma unroll
      for (int k = 0; k < 4; ++k) v[k] = fmaxf(v[k], 0.f);
    }
    reinterpret_cast<V*>(data)[i] = v;
  } else {
    float v = data[i];
    if (bias != nullptr) v += bias[i % features];
    if (relu) v = fmaxf(v, 0.f);
    data[i] = v;
  }
}

template <bool BLEND>
__global__ void __launch_bounds__(kThreads)
    scale_blend_kernel(float* data, const float* prior, float alpha,
                       float beta, size_t n) {
  const size_t i = static_cast<size_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (i >= n) return;
  // A zero factor drops its term outright (NaN or Inf in it do not survive),
  // as the reference does by skipping the convolution / zeroing the output.
  float v = alpha == 0.f ? 0.f : alpha * data[i];
  if (BLEND) v += beta * prior[i];
  data[i] = v;
}

}  // namespace

int launch_bias_act_f32(float* data, const float* bias, int features, size_t n,
                        bool relu, hipStream_t stream) {
  const bool vec = features % 4 == 0 && aligned16(data) &&
                   (bias == nullptr || aligned16(bias));
  if (vec) {
    const size_t n_vec = n / 4;
    hipLaunchKernelGGL(bias_act_kernel<true>,
                       dim3(static_cast<unsigned>(ceil_div(n_vec, size_t{kThreads}))),
                       dim3(kThreads), 0, stream, data, bias,
                       static_cast<unsigned>(features), n_vec, relu ? 1 : 0);
  } else {
    hipLaunchKernelGGL(bias_act_kernel<false>,
                       dim3(static_cast<unsigned>(ceil_div(n, size_t{kThreads}))),
                       dim3(kThreads), 0, stream, data, bias,
                       static_cast<unsigned>(features), n, relu ? 1 : 0);
  }
  const hipError_t e = hipGetLastError();
  return e == hipSuccess ? SNN_HIP_OK : report_hip_error(e, "bias_act_kernel");
}

int launch_scale_blend_f32(float* data, const float* prior, float alpha,
                           float beta, size_t n, hipStream_t stream) {
  const dim3 grid(static_cast<unsigned>(ceil_div(n, size_t{kThreads})));
  if (beta != 0.f && prior != nullptr)
    hipLaunchKernelGGL(scale_blend_kernel<true>, grid, dim3(kThreads), 0,
                       stream, data, prior, alpha, beta, n);
  else
    hipLaunchKernelGGL(scale_blend_kernel<false>, grid, dim3(kThreads), 0,
                       stream, data, prior, alpha, beta, n);
  const hipError_t e = hipGetLastError();
  return e == hipSuccess ? SNN_HIP_OK
                         : report_hip_error(e, "scale_blend_kernel");
}

int launch_pointwise_forward_f32(int op, const float* in, float* out, size_t n,
                                 hipStream_t stream) {
  return dispatch_pointwise<float, false>(op, in, nullptr, out, n, stream);
}
int launch_pointwise_forward_f16(int op, const _Float16* in, _Float16* out,
                                 size_t n, hipStream_t stream) {
  return dispatch_pointwise<_Float16, false>(op, in, nullptr, out, n, stream);
}
int launch_pointwise_grad_f32(int op, const float* val, const float* err,
                              float* out, size_t n, hipStream_t stream) {
  return dispatch_pointwise<float, true>(op, val, err, out, n, stream);
}
int launch_pointwise_grad_f16(int op, const _Float16* val, const _Float16* err,
                              _Float16* out, size_t n, hipStream_t stream) {
  return dispatch_pointwise<_Float16, true>(op, val, err, out, n, stream);
}
int launch_binaryop_f32(int op, const float* lhs, const float* rhs, float* out,
                        const int* lhs_dims, int n_lhs, const int* rhs_dims,
                        int n_rhs, hipStream_t stream) {
  return launch_binaryop_t<float>(op, lhs, rhs, out, lhs_dims, n_lhs, rhs_dims,
                                  n_rhs, stream);
}
int launch_binaryop_f16(int op, const _Float16* lhs, const _Float16* rhs,
                        _Float16* out, const int* lhs_dims, int n_lhs,
                        const int* rhs_dims, int n_rhs, hipStream_t stream) {
  return launch_binaryop_t<_Float16>(op, lhs, rhs, out, lhs_dims, n_lhs,
                                     rhs_dims, n_rhs, stream);
}

}  // namespace snn
