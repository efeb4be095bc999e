/*
 * CPU oracle -- see oracle.h.  TEST INFRASTRUCTURE ONLY; never linked into or
 * loaded by the shipped HIP library.
 */
#include "oracle.h"

#include <float.h>
#include <math.h>
#include <stddef.h>
#include <stdlib.h>
#ifdef _OPENMP
#include <omp.h>
#endif

static inline int imin(int a, int b) { return a < b ? a : b; }
static inline int imax(int a, int b) { return a > b ? a : b; }

/* First / one-past-last output index whose window [o*stride-pad,
 * o*stride-pad+window) contains input index i, clipped to [0, n_out). */
static inline int cover_begin(int i, int pad, int window, int stride) {
  const int t = i + pad - window + 1; /* smallest o*stride allowed */
  if (t <= 0) return 0;
  return (t + stride - 1) / stride;
}
static inline int cover_end(int i, int pad, int stride, int n_out) {
  return imin((i + pad) / stride + 1, n_out);
}

#define CAT2(a, b) a##b
#define CAT(a, b) CAT2(a, b)

#define ACC float
#define FN(name) CAT(name, _f32)
#include "oracle_body.inc"
#undef ACC
#undef FN

#define ACC double
#define FN(name) CAT(name, _f64)
#include "oracle_body.inc"
#undef ACC
#undef FN

int oracle_set_threads(int threads) {
#ifdef _OPENMP
  if (threads <= 0) threads = omp_get_num_procs();
  omp_set_num_threads(threads);
  return threads;
#else
  (void)threads;
  return 1;
#endif
}

/* include/portdnn/helpers/padding.h:51-69 */
void oracle_calculate_padding(int input, int window, int stride, int same,
                              int* padding, int* output) {
  if (same) {
    const int out = (input + stride - 1) / stride;
    const int needed = (out - 1) * stride + window - input;
    *output = out;
    /* C division truncates toward zero exactly as the reference's Index
     * division does when `needed` is negative. */
    *padding = needed / 2;
  } else {
    /* round_ratio_up of include/portdnn/helpers/ratio.h:70-79: rounds toward
     * +inf for a non-negative numerator, truncates a negative one. */
    const int num = input - window + 1;
    const int quotient = num / stride;
    *output = num < 0 ? quotient : quotient + (num % stride != 0);
    *padding = 0;
  }
}

#define DISPATCH(name, ...)    \
  do {                         \
    if (acc64)                 \
      name##_f64(__VA_ARGS__); \
    else                       \
      name##_f32(__VA_ARGS__); \
  } while (0)

void oracle_conv2d_forward(const float* in, const float* fil, float* out,
                           const oracle_params* p, int acc64) {
  DISPATCH(conv2d_forward, in, fil, out, p);
}
void oracle_conv2d_input_backprop(const float* dy, const float* fil, float* dx,
                                  const oracle_params* p, int acc64) {
  DISPATCH(conv2d_input_backprop, dy, fil, dx, p);
}
void oracle_conv2d_filter_backprop(const float* in, const float* dy, float* dw,
                                   const oracle_params* p, int acc64) {
  DISPATCH(conv2d_filter_backprop, in, dy, dw, p);
}
int oracle_conv2d_winograd_forward(const float* in, const float* fil,
                                   float* out, const oracle_params* p,
                                   int tile, int acc64) {
  if ((tile != 2 && tile != 4) || p->window_rows != 3 || p->window_cols != 3 ||
      p->stride_rows != 1 || p->stride_cols != 1)
    return 1;
  DISPATCH(conv2d_winograd_forward, in, fil, out, p, tile);
  return 0;
}
void oracle_depthwise_forward(const float* in, const float* fil, float* out,
                              const oracle_params* p, int acc64) {
  DISPATCH(depthwise_forward, in, fil, out, p);
}
void oracle_depthwise_input_backprop(const float* dy, const float* fil,
                                     float* dx, const oracle_params* p,
                                     int acc64) {
  DISPATCH(depthwise_input_backprop, dy, fil, dx, p);
}
void oracle_depthwise_filter_backprop(const float* in, const float* dy,
                                      float* dw, const oracle_params* p,
                                      int acc64) {
  DISPATCH(depthwise_filter_backprop, in, dy, dw, p);
}
void oracle_pool_avg_forward(const float* in, float* out,
                             const oracle_params* p, int acc64) {
  DISPATCH(pool_avg_forward, in, out, p);
}
void oracle_pool_avg_grad(const float* dy, float* dx, const oracle_params* p,
                          int acc64) {
  DISPATCH(pool_avg_grad, dy, dx, p);
}
void oracle_matmul(const float* a, const float* b, float* c, int batches, int m,
                   int k, int n, int trans_a, int trans_b, float beta,
                   int acc64) {
  DISPATCH(matmul, a, b, c, batches, m, k, n, trans_a, trans_b, beta);
}

/* Max pooling forward: src/pooling/kernels.h:61-99 with the scalar Max /
 * MaxWithNan operators of src/pooling/operators_impl.h:27-53.  Start value
 * numeric_limits<T>::lowest(); Max replaces only on `val > max` (so a NaN
 * never enters), MaxWithNan also replaces when val is NaN (and then stays NaN
 * unless a later NaN replaces it, because nothing compares greater than NaN). */
void oracle_pool_max_forward(const float* in, float* out,
                             const oracle_params* p, int nan_mode) {
  const int C = p->channels;
  const long n_pix = (long)p->batch * p->out_rows * p->out_cols;
#pragma omp parallel for schedule(static)
  for (long pix = 0; pix < n_pix; ++pix) {
    const int ox = (int)(pix % p->out_cols);
    const int oy = (int)((pix / p->out_cols) % p->out_rows);
    const int n = (int)(pix / ((long)p->out_cols * p->out_rows));
    const float* in_n = in + (long)n * p->in_rows * p->in_cols * C;
    int r0 = oy * p->stride_rows - p->pad_rows;
    const int r1 = imin(r0 + p->window_rows, p->in_rows);
    r0 = imax(r0, 0);
    int c0 = ox * p->stride_cols - p->pad_cols;
    const int c1 = imin(c0 + p->window_cols, p->in_cols);
    c0 = imax(c0, 0);
    for (int ch = 0; ch < C; ++ch) {
      float best = -FLT_MAX;
      for (int r = r0; r < r1; ++r) {
        for (int c = c0; c < c1; ++c) {
          const float v = in_n[((long)r * p->in_cols + c) * C + ch];
          if ((nan_mode && isnan(v)) || v > best) best = v;
        }
      }
      out[pix * C + ch] = best;
    }
  }
}

/* EqualCheck of src/pooling/operators_impl.h:89-113: Max compares with ==,
 * MaxWithNan additionally treats two NaNs as equal. */
static inline int pool_equal(float a, float b, int nan_mode) {
  if (nan_mode && isnan(a) && isnan(b)) return 1;
  return a == b;
}

/* Max pooling gradient: src/pooling/kernels.h:141-239.  Every dY element goes
 * to the FIRST element of its in-bounds window (row-major scan) that equals
 * the forward output. */
void oracle_pool_max_grad(const float* in, const float* out, const float* dy,
                          float* dx, const oracle_params* p, int nan_mode) {
  const int C = p->channels;
  const long n_in = (long)p->batch * p->in_rows * p->in_cols * C;
  for (long i = 0; i < n_in; ++i) dx[i] = 0.0f;
  const long n_pix = (long)p->batch * p->out_rows * p->out_cols;
  /* Serial over output pixels of one image keeps "+=" race free; images are
   * independent. */
#pragma omp parallel for schedule(static)
  for (int n = 0; n < p->batch; ++n) {
    const float* in_n = in + (long)n * p->in_rows * p->in_cols * C;
    float* dx_n = dx + (long)n * p->in_rows * p->in_cols * C;
    for (int oy = 0; oy < p->out_rows; ++oy) {
      int r0 = oy * p->stride_rows - p->pad_rows;
      const int r1 = imin(r0 + p->window_rows, p->in_rows);
      r0 = imax(r0, 0);
      for (int ox = 0; ox < p->out_cols; ++ox) {
        int c0 = ox * p->stride_cols - p->pad_cols;
        const int c1 = imin(c0 + p->window_cols, p->in_cols);
        c0 = imax(c0, 0);
        const long opix = ((long)n * p->out_rows + oy) * p->out_cols + ox;
        for (int ch = 0; ch < C; ++ch) {
          const float target = out[opix * C + ch];
          int done = 0;
          for (int r = r0; r < r1 && !done; ++r) {
            for (int c = c0; c < c1 && !done; ++c) {
              const long idx = ((long)r * p->in_cols + c) * C + ch;
              if (pool_equal(in_n[idx], target, nan_mode)) {
                dx_n[idx] += dy[opix * C + ch];
                done = 1;
              }
            }
          }
        }
      }
    }
  }
  (void)n_pix;
}

/* Tiled forward: src/conv2d/tiled/kernels.h:99-190 with the generic tile list
 * entry of src/conv2d/tiled/launch_tiled.cc:215-226 (2x2 output tile, channel
 * vector 1, feature vector 4).  Work-item = (batch, tile row, tile col,
 * feature vector), un-flattened in that order (kernels.h:107-114); per item:
 * for each channel, load the R x S x 1 x 4 filter tile, then for each of the
 * (2-1)*stride+R input rows load a row strip of (2-1)*stride+S values
 * (zero outside the image, tiles.h:57-110) and mad it into every output row /
 * column / filter column it touches (kernels.h:149-190).  Output writes are
 * clipped to the image (tiles.h, OutputTile::write_out). */
#define TILE_R 2
#define TILE_C 2
#define FVEC 4
#define MAX_WIN 3
#define MAX_STRIP ((TILE_C - 1) * 2 + MAX_WIN)

int oracle_conv2d_tiled_forward(const float* in, const float* fil, float* out,
                                const oracle_params* p, int threads) {
  const int R = p->window_rows, S = p->window_cols;
  const int st = p->stride_rows;
  if (R != S || (R != 1 && R != 3)) return 1;
  if (p->stride_cols != st || (st != 1 && st != 2)) return 1;
  if (p->features % FVEC) return 1;
  oracle_set_threads(threads);
  const int C = p->channels, K = p->features;
  const int n_tile_rows = (p->out_rows + TILE_R - 1) / TILE_R;
  const int n_tile_cols = (p->out_cols + TILE_C - 1) / TILE_C;
  const int n_fvec = K / FVEC;
  const int in_tile_rows = (TILE_R - 1) * st + R;
  const int in_tile_cols = (TILE_C - 1) * st + S;
  const long n_items = (long)p->batch * n_tile_rows * n_tile_cols * n_fvec;
#pragma omp parallel for schedule(static)
  for (long item = 0; item < n_items; ++item) {
    const int feature = (int)(item % n_fvec) * FVEC;
    const int col_idx = (int)((item / n_fvec) % n_tile_cols) * TILE_C;
    const int row_idx =
        (int)((item / ((long)n_fvec * n_tile_cols)) % n_tile_rows) * TILE_R;
    const int batch = (int)(item / ((long)n_fvec * n_tile_cols * n_tile_rows));
    const int cstart = col_idx * st - p->pad_cols;
    const int rstart = row_idx * st - p->pad_rows;
    float acc[TILE_R][TILE_C][FVEC] = {{{0}}};
    const float* in_n = in + (long)batch * p->in_rows * p->in_cols * C;
    for (int ch = 0; ch < C; ++ch) {
      float ftile[MAX_WIN][MAX_WIN][FVEC];
      for (int r = 0; r < R; ++r)
        for (int s = 0; s < S; ++s)
          for (int v = 0; v < FVEC; ++v)
            ftile[r][s][v] = fil[((long)(r * S + s) * C + ch) * K + feature + v];
      for (int i = 0; i < in_tile_rows; ++i) {
        const int y = rstart + i;
        if (y < 0 || y >= p->in_rows) continue;
        float strip[MAX_STRIP];
        for (int j = 0; j < in_tile_cols; ++j) {
          const int x = cstart + j;
          strip[j] = (x < 0 || x >= p->in_cols)
                         ? 0.0f
                         : in_n[((long)y * p->in_cols + x) * C + ch];
        }
        for (int orow = 0; orow < TILE_R; ++orow) {
          const int frow = i - orow * st;
          if (frow < 0 || frow >= R) continue;
          for (int ocol = 0; ocol < TILE_C; ++ocol) {
            for (int fcol = 0; fcol < S; ++fcol) {
              const float x = strip[ocol * st + fcol];
              for (int v = 0; v < FVEC; ++v) {
                acc[orow][ocol][v] =
                    fmaf(x, ftile[frow][fcol][v], acc[orow][ocol][v]);
              }
            }
          }
        }
      }
    }
    for (int orow = 0; orow < TILE_R; ++orow) {
      const int oy = row_idx + orow;
      if (oy >= p->out_rows) continue;
      for (int ocol = 0; ocol < TILE_C; ++ocol) {
        const int ox = col_idx + ocol;
        if (ox >= p->out_cols) continue;
        float* o = out + (((long)batch * p->out_rows + oy) * p->out_cols + ox) * K +
                   feature;
        for (int v = 0; v < FVEC; ++v) o[v] = acc[orow][ocol][v];
      }
    }
  }
  return 0;
}

/* src/pointwise/kernels.h: Relu<Forward> :47-49 max(val, 0); Tanh :69-71;
 * Exp :91-93; Log :116-118; Floor :137-139; Sqrt :152-154. */
int oracle_pointwise_forward(int op, const float* in, float* out, long n) {
  for (long i = 0; i < n; ++i) {
    const float v = in[i];
    switch (op) {
      case ORACLE_RELU: out[i] = fmaxf(v, 0.0f); break;
      case ORACLE_TANH: out[i] = tanhf(v); break;
      case ORACLE_EXP: out[i] = expf(v); break;
      case ORACLE_LOG: out[i] = logf(v); break;
      case ORACLE_FLOOR: out[i] = floorf(v); break;
      case ORACLE_SQRT: out[i] = sqrtf(v); break;
      default: return 1;
    }
  }
  return 0;
}

/* src/pointwise/kernels.h: Relu<Gradient> :53-57 select(0, err, val > 0);
 * Tanh :75-77 (1 - val*val) * err; Exp :100-102 exp(val) + err (as written
 * there); Log :122-124 (1 / val) * err; Sqrt :158-160 (0.5 / val) * err. */
int oracle_pointwise_grad(int op, const float* val, const float* err,
                          float* out, long n) {
  for (long i = 0; i < n; ++i) {
    const float v = val[i], e = err[i];
    switch (op) {
      case ORACLE_RELU: out[i] = v > 0.0f ? e : 0.0f; break;
      case ORACLE_TANH: out[i] = (1.0f - v * v) * e; break;
      case ORACLE_EXP: out[i] = expf(v) + e; break;
      case ORACLE_LOG: out[i] = (1.0f / v) * e; break;
      case ORACLE_SQRT: out[i] = (0.5f / v) * e; break;
      default: return 1;
    }
  }
  return 0;
}

/* include/portdnn/internal/binaryop/launch.h:40-62 (output shape) and
 * src/binaryop/kernels.h:86-124 (index arithmetic of the general kernel). */
int oracle_binaryop(int op, const float* lhs, const float* rhs, float* out,
                    const int* lhs_dims, int n_lhs, const int* rhs_dims,
                    int n_rhs) {
  int l[4] = {1, 1, 1, 1}, r[4] = {1, 1, 1, 1}, o[4];
  if (n_lhs > 4 || n_rhs > 4 || n_lhs < 0 || n_rhs < 0) return 1;
  for (int i = 0; i < n_lhs; ++i) l[4 - n_lhs + i] = lhs_dims[i];
  for (int i = 0; i < n_rhs; ++i) r[4 - n_rhs + i] = rhs_dims[i];
  for (int i = 0; i < 4; ++i) {
    if (l[i] < 1 || r[i] < 1) return 1;
    if (l[i] != r[i] && l[i] != 1 && r[i] != 1) return 1;
    o[i] = l[i] > r[i] ? l[i] : r[i];
  }
  const long total = (long)o[0] * o[1] * o[2] * o[3];
  for (long idx = 0; idx < total; ++idx) {
    long rem = idx, li = 0, ri = 0, ls = 1, rs = 1;
    for (int d = 3; d >= 0; --d) {
      const long c = d > 0 ? rem % o[d] : rem;
      if (c < l[d]) li += c * ls;
      if (c < r[d]) ri += c * rs;
      ls *= l[d];
      rs *= r[d];
      if (d > 0) rem /= o[d];
    }
    const float a = lhs[li], b = rhs[ri];
    switch (op) {
      case ORACLE_ADD: out[idx] = a + b; break;
      case ORACLE_SUB: out[idx] = a - b; break;
      case ORACLE_MUL: out[idx] = a * b; break;
      case ORACLE_DIV: out[idx] = a / b; break;
      default: return 1;
    }
  }
  return 0;
}
