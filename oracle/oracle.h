/*
 * CPU oracle for the convolution / depthwise / pooling path.
 *
 * TEST INFRASTRUCTURE ONLY: this library is the checker the HIP kernels are
 * compared against and the CPU baseline that is timed beside them.  Nothing in
 * the shipped library links, loads or calls it.
 *
 * Every function restates, in plain C, what the corresponding portDNN kernel
 * computes (reference file:line cited per function in oracle.c).  Layouts:
 * tensors NHWC row-major, dense filter HWCF [R][S][C][K], depthwise filter
 * [R][S][C][multiplier] with output channel c*multiplier+j.
 *
 * How each function is pinned (nothing here is "parity unpinned"):
 *   conv2d fwd/inbk/filbk, depthwise fwd/inbk/filbk, max/avg pool fwd+grad:
 *     the reference's generated golden vectors (tests/golden/ *.npz, exact
 *     integers) -- tests/test_oracle_golden.py.
 *   max-pool NaN rules: the hand-written cases of
 *     test/pooling/max_pooling_with_nan.cc -- tests/test_oracle_golden.py.
 *   padding helper: known answers of test/helpers/padding.cc.
 *   tiled forward: must equal the direct forward bit-for-bit on integer data
 *     and is checked against the same goldens.
 *   matmul: textbook definition, checked against numpy float64 matmul for all
 *     transpose/beta combinations.
 *   Winograd forward (F(2x2,3x3) and F(4x4,3x3), the reference's transform
 *     matrices): with double accumulation it must equal the direct
 *     convolution to ~1e-12 on random data and exactly on the integer goldens
 *     (tests/test_oracle_golden.py); the float variant is the same code.
 *   pointwise (relu, tanh, log, floor, sqrt; forward and gradient) and
 *     binaryop (add, sub, mul, div with broadcasting): the reference's golden
 *     vectors of test/pointwise/ *.cc and test/binaryop/ *.cc
 *     (tests/golden/pointwise.npz, binaryop.npz).  The reference holds no
 *     vectors for exp: it is pinned against libm's exp (forward) and the
 *     identity exp(val) + err the reference kernel computes (gradient).
 */
#ifndef PORTDNN_AMD_ORACLE_H_
#define PORTDNN_AMD_ORACLE_H_

#ifdef __cplusplus
extern "C" {
#endif

/* One record serves conv2d, depthwise (features = channel multiplier) and
 * pooling (features ignored). */
typedef struct oracle_params {
  int channels;
  int features;
  int batch;
  int in_rows, in_cols;
  int window_rows, window_cols;
  int stride_rows, stride_cols;
  int out_rows, out_cols;
  int pad_rows, pad_cols;
} oracle_params;

/* include/portdnn/helpers/padding.h:51-69.  same != 0 selects SAME. */
void oracle_calculate_padding(int input, int window, int stride, int same,
                              int* padding, int* output);

/* acc64 != 0 accumulates in double and rounds once at the end (the
 * "mathematically exact" answer used for tolerance checks); acc64 == 0
 * accumulates in float in the reference's loop order. */
void oracle_conv2d_forward(const float* in, const float* fil, float* out,
                           const oracle_params* p, int acc64);
/* The same result by the Winograd algorithm with tile x tile output blocks
 * (2: Algorithm::Winograd, 4: Algorithm::WinogradLarge), 3x3 stride 1 only;
 * every stage in float (acc64 == 0) or double.  Returns non-zero for other
 * shapes.  include/portdnn/internal/conv2d/winograd/launch.h:63-264,
 * src/conv2d/winograd/kernels/tiles_impl.h:70-198,774-1000. */
int oracle_conv2d_winograd_forward(const float* in, const float* fil,
                                   float* out, const oracle_params* p,
                                   int tile, int acc64);
void oracle_conv2d_input_backprop(const float* dy, const float* fil, float* dx,
                                  const oracle_params* p, int acc64);
void oracle_conv2d_filter_backprop(const float* in, const float* dy, float* dw,
                                   const oracle_params* p, int acc64);

/* portDNN's Tiled forward with the generic tile list entry
 * (window, stride, 2 rows, 2 cols, channel vector 1, feature vector 4):
 * one "work-item" per 2x2x4 output tile, float mad, channel-outermost
 * accumulation.  Requires window 1 or 3 (square), stride 1 or 2 and
 * features % 4 == 0; returns non-zero otherwise.  threads <= 0 uses every
 * host core. */
int oracle_conv2d_tiled_forward(const float* in, const float* fil, float* out,
                                const oracle_params* p, int threads);

void oracle_depthwise_forward(const float* in, const float* fil, float* out,
                              const oracle_params* p, int acc64);
void oracle_depthwise_input_backprop(const float* dy, const float* fil,
                                     float* dx, const oracle_params* p,
                                     int acc64);
void oracle_depthwise_filter_backprop(const float* in, const float* dy,
                                      float* dw, const oracle_params* p,
                                      int acc64);

/* nan_mode 0: pooling::Max (scalar form: NaN inputs never win);
 * nan_mode 1: pooling::MaxWithNan (a NaN in the window wins). */
void oracle_pool_max_forward(const float* in, float* out,
                             const oracle_params* p, int nan_mode);
void oracle_pool_avg_forward(const float* in, float* out,
                             const oracle_params* p, int acc64);
/* in: forward input, out: forward output, dy: gradient w.r.t. out,
 * dx: gradient w.r.t. in (written). */
void oracle_pool_max_grad(const float* in, const float* out, const float* dy,
                          float* dx, const oracle_params* p, int nan_mode);
void oracle_pool_avg_grad(const float* dy, float* dx, const oracle_params* p,
                          int acc64);

/* Batched row-major GEMM  C[b] = op(A[b]) * op(B[b]) + beta * C[b]
 * with op(A) m x k, op(B) k x n. */
void oracle_matmul(const float* a, const float* b, float* c, int batches, int m,
                   int k, int n, int trans_a, int trans_b, float beta,
                   int acc64);

/* Element-wise operators of src/pointwise/kernels.h:36-153. */
enum {
  ORACLE_RELU = 0, ORACLE_TANH = 1, ORACLE_EXP = 2, ORACLE_LOG = 3,
  ORACLE_FLOOR = 4, ORACLE_SQRT = 5
};
/* out[i] = op(in[i]).  Returns non-zero for an unknown operator. */
int oracle_pointwise_forward(int op, const float* in, float* out, long n);
/* out[i] = op'(val[i], err[i]) with the reference's meaning of `val`: the
 * forward OUTPUT for relu / tanh / exp / sqrt, the forward INPUT for log
 * (test/pointwise/pointwise_fixture.h:115-124).  Floor has no gradient. */
int oracle_pointwise_grad(int op, const float* val, const float* err,
                          float* out, long n);

/* Broadcasting binary operators of src/binaryop/kernels.h:33-124:
 * dimensions are right-aligned, missing leading ones are 1, a dimension of 1
 * broadcasts.  n_lhs, n_rhs <= 4 (0 = scalar).  Returns non-zero when the
 * shapes do not broadcast. */
enum { ORACLE_ADD = 0, ORACLE_SUB = 1, ORACLE_MUL = 2, ORACLE_DIV = 3 };
int oracle_binaryop(int op, const float* lhs, const float* rhs, float* out,
                    const int* lhs_dims, int n_lhs, const int* rhs_dims,
                    int n_rhs);

/* Thread count used by the OpenMP loops (<= 0: all cores). Returns the count
 * now in force. */
int oracle_set_threads(int threads);

#ifdef __cplusplus
}
#endif
#endif /* PORTDNN_AMD_ORACLE_H_ */
