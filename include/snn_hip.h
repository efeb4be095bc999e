/*
 * C ABI of libsnn_hip.so -- the MI355X (gfx950) implementation of portDNN's
 * convolution / depthwise-convolution / pooling hot path.
 *
 * portDNN itself has no C ABI: its boundary is a set of header templates
 * (include/portdnn/<op>/launch.h) over explicitly instantiated launchers that
 * live in libportdnn (src/<op>/launch*.cc).  The entry points below are what a
 * HIP backend for those templates binds, one per (operator, direction, data
 * type); each comment names the reference interface it stands in for.  The
 * C++ drop-in templates in include/portdnn/ are a thin layer over this file.
 *
 * Conventions
 *  - All tensor pointers are DEVICE pointers.  Tensors are NHWC row-major;
 *    dense filters are HWCF [R][S][C][K]; depthwise filters are
 *    [R][S][C][multiplier] and output channel c*multiplier+j.
 *  - `stream` is a hipStream_t passed as void* (NULL = the default stream).
 *    Every call is asynchronous and stream-ordered; no call synchronises.
 *  - The return value is a snn_hip_status.  Values 0..5 are portDNN's
 *    StatusCode enumerators in declaration order
 *    (include/portdnn/status.h:31-44); 6 reports a HIP runtime failure.
 *  - Workspace sizes are counted in ELEMENTS of the data type, as in
 *    include/portdnn/conv2d/workspace_size.h:42-47.
 *  - f16 entry points take IEEE binary16 data and accumulate in fp32.
 */
#ifndef SNN_HIP_H_
#define SNN_HIP_H_

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

#if defined(_WIN32)
#define SNN_HIP_API
#else
#define SNN_HIP_API __attribute__((visibility("default")))
#endif

typedef enum snn_hip_status {
  SNN_HIP_OK = 0,
  SNN_HIP_INVALID_ALGORITHM = 1,
  SNN_HIP_INDEX_EXCEEDED = 2,
  SNN_HIP_INSUFFICIENT_WORKSPACE = 3,
  SNN_HIP_ALLOCATION_PROBLEM = 4,
  SNN_HIP_INVALID_PARAMETER = 5,
  SNN_HIP_DEVICE_ERROR = 6
} snn_hip_status;

/* sycldnn::conv2d::Algorithm, include/portdnn/conv2d/algorithm.h:30-45 */
typedef enum snn_hip_algorithm {
  SNN_HIP_ALGO_NOT_SUPPORTED = 0,
  SNN_HIP_ALGO_DIRECT = 1,
  SNN_HIP_ALGO_TILED = 2,
  SNN_HIP_ALGO_IM2COL = 3,
  SNN_HIP_ALGO_WINOGRAD = 4,
  SNN_HIP_ALGO_WINOGRAD_LARGE = 5,
  SNN_HIP_ALGO_MATMUL = 6
} snn_hip_algorithm;

/* sycldnn::conv2d::conv_type tags, include/portdnn/conv2d/conv_type.h:35-47 */
typedef enum snn_hip_direction {
  SNN_HIP_FORWARD = 0,
  SNN_HIP_INPUT_BACKPROP = 1,
  SNN_HIP_FILTER_BACKPROP = 2
} snn_hip_direction;

/* POD image of sycldnn::conv2d::Conv2DParams
 * (include/portdnn/conv2d/params.h:32-112), same field order.  The three
 * format fields hold the enumerator values of DataFormat (NHWC = 0, NCHW = 1),
 * FilterFormat (HWCF = 0, FCHW = 1, FHWC = 2) and BatchFormat (STRIDED = 0,
 * INTERLEAVED = 1); only the first of each is accepted. */
typedef struct snn_hip_conv2d_params {
  int channels;
  int features;
  int batch;
  int in_rows;
  int in_cols;
  int window_rows;
  int window_cols;
  int stride_rows;
  int stride_cols;
  int out_rows;
  int out_cols;
  int pad_rows;
  int pad_cols;
  int dilation_rows;
  int dilation_cols;
  int groups;
  int input_format;
  int filter_format;
  int group_format;
} snn_hip_conv2d_params;

/* POD image of sycldnn::depthwise_conv2d::DepthwiseConv2DParams
 * (include/portdnn/depthwise_conv2d/params.h:33-94). */
typedef struct snn_hip_depthwise_params {
  int channels;
  int channel_multiplier;
  int batch;
  int in_rows;
  int in_cols;
  int window_rows;
  int window_cols;
  int stride_rows;
  int stride_cols;
  int out_rows;
  int out_cols;
  int pad_rows;
  int pad_cols;
  int input_format;
  int filter_format;
} snn_hip_depthwise_params;

/* POD image of sycldnn::pooling::PoolingParams
 * (include/portdnn/pooling/params.h:30-73). */
typedef struct snn_hip_pooling_params {
  int in_rows;
  int in_cols;
  int out_rows;
  int out_cols;
  int window_rows;
  int window_cols;
  int stride_rows;
  int stride_cols;
  int batch;
  int channels;
  int pad_rows;
  int pad_cols;
  int input_format;
} snn_hip_pooling_params;

/* sycldnn::pooling operators, include/portdnn/pooling/operators.h:23-42 */
typedef enum snn_hip_pool_op {
  SNN_HIP_POOL_MAX = 0,
  SNN_HIP_POOL_MAX_WITH_NAN = 1,
  SNN_HIP_POOL_AVERAGE = 2
} snn_hip_pool_op;

/* ---- library ------------------------------------------------------------ */

/* Library version, major*10000 + minor*100 + patch. */
SNN_HIP_API int snn_hip_version(void);
/* Static, human-readable name of a status value. */
SNN_HIP_API const char* snn_hip_status_string(int status);
/* Text of the last HIP runtime error seen by the calling thread ("" if none). */
SNN_HIP_API const char* snn_hip_last_error(void);

/* Kernel timing for benchmarks (no counterpart in the reference, whose
 * launches return a cl::sycl::event that carries profiling information).
 * While enabled, every convolution launch brackets its dominant kernel -- the
 * implicit-GEMM or fused Winograd kernel, not the filter preparation or zero
 * fill around it -- with HIP events recorded on the launch stream; depthwise
 * and pooling launches bracket everything they enqueue.
 * snn_hip_kernel_timing_read waits for the recorded events, returns the summed
 * kernel time in milliseconds and the number of kernels, and clears the
 * record.  Launches from several threads may record concurrently (the record
 * is mutex-guarded and stops growing at 65536 kernels until it is read); a
 * read waits for every recorded kernel, so call it from one thread once the
 * timed launches have been enqueued. */
SNN_HIP_API int snn_hip_kernel_timing_enable(int enable);
SNN_HIP_API int snn_hip_kernel_timing_read(double* total_ms, int* kernels);

/* Diagnostics for the stream-ordered temporaries some launches take when the
 * caller passes no workspace (no counterpart in portDNN, whose temporaries
 * come from backend.allocate): bytes currently reserved by, and the high-water
 * mark of bytes in use in, the two pools such temporaries come from on the
 * current device -- the library's own pool and the device's default pool.
 * With reset_high != 0 the high-water marks are cleared after reading, so a
 * caller can bracket a sequence of launches and see whether any of them took
 * a temporary. */
SNN_HIP_API int snn_hip_temporary_memory_stats(
    unsigned long long* reserved_bytes, unsigned long long* used_high_bytes,
    int reset_high);

/* ---- dense convolution ---------------------------------------------------
 * Stand-ins for sycldnn::conv2d::internal::launch_{direct,tiled,matmul,
 * im2col,winograd} reached from sycldnn::conv2d::launch<T, ConvType>
 * (include/portdnn/conv2d/launch.h:59-118 via
 * include/portdnn/internal/conv2d/launch.h:99-207): validate the parameters,
 * check that `algorithm` supports them (SNN_HIP_INVALID_ALGORITHM otherwise,
 * as internal/conv2d/launch.h:127-129,191-197) and enqueue the kernels.
 *
 * forward:         input  [N,H,W,C]    filter [R,S,C,K]    output [N,OH,OW,K]
 * input_backprop:  input = dY [N,OH,OW,K], filter [R,S,C,K], output = dX [N,H,W,C]
 * filter_backprop: input = X [N,H,W,C], filter = dY [N,OH,OW,K], output = dW [R,S,C,K]
 * (operand roles of include/portdnn/conv2d/sizes.h:166-179).
 *
 * `workspace` may be NULL with workspace_elems == 0.  Winograd then returns
 * SNN_HIP_INSUFFICIENT_WORKSPACE (internal/conv2d/winograd/launch.h:271-286);
 * the other algorithms need no caller scratch. */
SNN_HIP_API int snn_hip_conv2d_forward_f32(
    const float* input, const float* filter, float* output,
    const snn_hip_conv2d_params* params, int algorithm, float* workspace,
    size_t workspace_elems, void* stream);
SNN_HIP_API int snn_hip_conv2d_input_backprop_f32(
    const float* input, const float* filter, float* output,
    const snn_hip_conv2d_params* params, int algorithm, float* workspace,
    size_t workspace_elems, void* stream);
SNN_HIP_API int snn_hip_conv2d_filter_backprop_f32(
    const float* input, const float* filter, float* output,
    const snn_hip_conv2d_params* params, int algorithm, float* workspace,
    size_t workspace_elems, void* stream);
SNN_HIP_API int snn_hip_conv2d_forward_f16(
    const void* input, const void* filter, void* output,
    const snn_hip_conv2d_params* params, int algorithm, void* workspace,
    size_t workspace_elems, void* stream);
/* The two gradients in half precision (fp32 accumulation), the reference's
 * launch<half, conv_type::InputBackprop / FilterBackprop>.  With channel
 * counts in multiples of 64 they run on the matrix cores (3x3 stride-1 SAME
 * and 1x1 filter gradients and stride-1 input gradients on binary16 matrix
 * instructions, other shapes on fp32 matrix instructions fed binary16
 * operands); shapes off those multiples run on the direct kernels.  No
 * half-precision launch requires a workspace; one of the size
 * snn_hip_conv2d_workspace_size_for reports saves a stream-ordered
 * temporary. */
SNN_HIP_API int snn_hip_conv2d_input_backprop_f16(
    const void* input, const void* filter, void* output,
    const snn_hip_conv2d_params* params, int algorithm, void* workspace,
    size_t workspace_elems, void* stream);
SNN_HIP_API int snn_hip_conv2d_filter_backprop_f16(
    const void* input, const void* filter, void* output,
    const snn_hip_conv2d_params* params, int algorithm, void* workspace,
    size_t workspace_elems, void* stream);

/* Run-to-run reproducibility.  The reference's kernels add every output's
 * terms in one fixed order, so its results repeat bit for bit.  The entry
 * points above do not always: where a launch would otherwise fill only part
 * of the GPU they split a reduction across work-groups whose partial sums
 * meet through float atomics -- the implicit-GEMM filter gradient (Im2col /
 * Tiled / Direct-fallback tags) always, except for the 7x7 stride-2
 * three-channel stem from 224 output rows over the batch upwards and for
 * every other layer with at least 32 channels, or with window size x channels
 * above 192, or with a feature count that is not a multiple of 4 (16-byte
 * aligned operands, at least 256 output pixels), whose partial filters are
 * summed in a fixed order; forward and input gradients of small
 * problems (fewer than ~640 64x64 output tiles, unless one of the kernels
 * that sum their parts in a fixed order takes the launch: stride-1 layers
 * with channels in multiples of 128, forward problems of fewer than 128
 * tiles) and the fused Winograd
 * kernel below 128 work units -- and the order of those additions, hence the
 * last bits of the result, can change between runs.  The Winograd filter
 * gradient and every launch without such a split are reproducible.
 *
 * snn_hip_conv2d_deterministic_f32 is the same operation as the three fp32
 * entry points (`direction` is a snn_hip_direction) with a fixed order of
 * additions: no reduction splits (small problems run on fewer work-groups),
 * and a filter gradient outside the Winograd algorithm runs on the direct
 * kernel, one lane per filter element (the layers named above keep their
 * kernel).  Two calls with the same arguments
 * return bit-identical results.  Workspace sizes are those of
 * snn_hip_conv2d_workspace_size. */
SNN_HIP_API int snn_hip_conv2d_deterministic_f32(
    int direction, const float* input, const float* filter, float* output,
    const snn_hip_conv2d_params* params, int algorithm, float* workspace,
    size_t workspace_elems, void* stream);

/* A launch in two calls, for callers that run many launches with one filter
 * (inference).  No counterpart in portDNN, whose Winograd launch transforms
 * the filter every time (internal/conv2d/winograd/launch.h:212-235).
 *
 * snn_hip_conv2d_prepare_filter_f32 writes into `workspace` whatever a launch
 * with these parameters, direction and algorithm derives from the filter
 * alone -- today the transformed filter of the fused Winograd forward /
 * input-gradient kernels; for every other path it does nothing and returns
 * SNN_HIP_OK.  snn_hip_conv2d_prepared_f32 is then the same operation as the
 * three fp32 entry points, except that it trusts those contents instead of
 * recomputing them: the caller guarantees that `workspace` (same pointer,
 * same size) still holds what a prepare call with the same filter values,
 * parameters, direction and algorithm wrote, and that nothing else wrote to
 * its first 16 * C * K elements since.  The one-call entry points never
 * trust a workspace: they always transform the filter they are given. */
SNN_HIP_API int snn_hip_conv2d_prepare_filter_f32(
    int direction, const float* filter, const snn_hip_conv2d_params* params,
    int algorithm, float* workspace, size_t workspace_elems, void* stream);
SNN_HIP_API int snn_hip_conv2d_prepared_f32(
    int direction, const float* input, const float* filter, float* output,
    const snn_hip_conv2d_params* params, int algorithm, float* workspace,
    size_t workspace_elems, void* stream);

/* sycldnn::conv2d::query_workspace_size<ConvType>(params, selector)
 * (include/portdnn/conv2d/workspace_size.h:158-163) for an already selected
 * algorithm.  Sizes in elements. */
SNN_HIP_API int snn_hip_conv2d_workspace_size(
    const snn_hip_conv2d_params* params, int direction, int algorithm,
    size_t* required_elems, size_t* recommended_elems);

/* The same for a given element type (a snn_hip_dtype), in elements of that
 * type.  portDNN's query does not know the element type
 * (workspace_size.h:158-163 takes only the parameters and the selector); the
 * half-precision kernels here are different kernels with different needs, so
 * a caller that sizes its scratch from the fp32 answer would allocate the
 * F(2x2,3x3) transform buffers for a launch that uses a filter-sized block.
 * For SNN_HIP_DTYPE_F16 `required` is always 0 (a launch without scratch
 * takes a stream-ordered temporary) and `recommended` is what the launch
 * uses.  SNN_HIP_DTYPE_F32 answers as snn_hip_conv2d_workspace_size. */
typedef enum snn_hip_dtype {
  SNN_HIP_DTYPE_F32 = 0,
  SNN_HIP_DTYPE_F16 = 1
} snn_hip_dtype;
SNN_HIP_API int snn_hip_conv2d_workspace_size_for(
    const snn_hip_conv2d_params* params, int direction, int algorithm,
    int dtype, size_t* required_elems, size_t* recommended_elems);

/* Does `algorithm` support these parameters in this direction?  Mirrors the
 * concrete selectors (include/portdnn/conv2d/selector/{tiled,winograd,matmul}_
 * selector.h, constant_selector.h): returns `algorithm` if it does, else
 * SNN_HIP_ALGO_NOT_SUPPORTED. */
SNN_HIP_API int snn_hip_conv2d_algorithm_supports(
    const snn_hip_conv2d_params* params, int direction, int algorithm);

/* The algorithm sycldnn::conv2d::get_default_selector(device) would pick on
 * this device (src/conv2d/selector/default_selector.cc:257-286), tuned for
 * MI355X. */
SNN_HIP_API int snn_hip_conv2d_default_algorithm(
    const snn_hip_conv2d_params* params, int direction);
/* The same for a given element type: half precision has no Winograd kernels,
 * so its 3x3 layers get the Tiled (forward) / Im2col tag, whose kernels and
 * workspace snn_hip_conv2d_workspace_size_for describes. */
SNN_HIP_API int snn_hip_conv2d_default_algorithm_for(
    const snn_hip_conv2d_params* params, int direction, int dtype);

/* ---- depthwise convolution -----------------------------------------------
 * Stand-ins for sycldnn::depthwise_conv2d::internal::launch<ConvType>
 * (src/depthwise_conv2d/launch.cc:100-121) reached from
 * sycldnn::depthwise_conv2d::launch (include/portdnn/depthwise_conv2d/
 * launch.h:54-91).  Operand roles as for the dense convolution with
 * K = C * multiplier. */
SNN_HIP_API int snn_hip_depthwise_conv2d_forward_f32(
    const float* input, const float* filter, float* output,
    const snn_hip_depthwise_params* params, void* stream);
SNN_HIP_API int snn_hip_depthwise_conv2d_input_backprop_f32(
    const float* input, const float* filter, float* output,
    const snn_hip_depthwise_params* params, void* stream);
SNN_HIP_API int snn_hip_depthwise_conv2d_filter_backprop_f32(
    const float* input, const float* filter, float* output,
    const snn_hip_depthwise_params* params, void* stream);
/* The fp32 filter gradient for callers that cannot allocate device memory
 * (code under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc).  No counterpart in the reference.  Same operands and result as
 * snn_hip_depthwise_conv2d_filter_backprop_f32, whose large-input path keeps
 * the work-groups' partial filters in a stream-ordered temporary; here they
 * live in a 9 MiB device array inside the library (held by every GPU the
 * library runs on until the process ends), sized for the largest plan that
 * path makes, so no hipMalloc / hipFree in any form is called.  A shape whose
 * partial filters would not fit is rejected with SNN_HIP_INVALID_PARAMETER
 * and a message in snn_hip_last_error().  All calls on one GPU share that
 * array: calls that overlap on one GPU (different streams or threads) race;
 * stream-ordered calls are safe.  The stream's device must be current.  The
 * first call on each device looks the array's address up
 * (hipGetSymbolAddress, which may load the library's device code): make one
 * call per device before a stream capture begins; later calls only enqueue
 * kernels. */
SNN_HIP_API int snn_hip_depthwise_conv2d_filter_backprop_noalloc_f32(
    const float* input, const float* filter, float* output,
    const snn_hip_depthwise_params* params, void* stream);
SNN_HIP_API int snn_hip_depthwise_conv2d_forward_f16(
    const void* input, const void* filter, void* output,
    const snn_hip_depthwise_params* params, void* stream);
SNN_HIP_API int snn_hip_depthwise_conv2d_input_backprop_f16(
    const void* input, const void* filter, void* output,
    const snn_hip_depthwise_params* params, void* stream);
SNN_HIP_API int snn_hip_depthwise_conv2d_filter_backprop_f16(
    const void* input, const void* filter, void* output,
    const snn_hip_depthwise_params* params, void* stream);

/* ---- pooling -------------------------------------------------------------
 * Stand-ins for sycldnn::pooling::internal::launch_pooling
 * (src/pooling/launch_pooling.cc:146-165) reached from
 * sycldnn::pooling::launch<T, PoolType, Direction>
 * (include/portdnn/pooling/launch.h:112-128 forward, :153-172 max gradient).
 * `op` is a snn_hip_pool_op. */
SNN_HIP_API int snn_hip_pooling_forward_f32(
    const float* input, float* output, const snn_hip_pooling_params* params,
    int op, void* stream);
SNN_HIP_API int snn_hip_pooling_forward_f16(
    const void* input, void* output, const snn_hip_pooling_params* params,
    int op, void* stream);
/* Max / MaxWithNan gradient: input_data and output_data are the forward
 * tensors, input_backprop is dY [N,OH,OW,C], output_backprop is dX [N,H,W,C]. */
SNN_HIP_API int snn_hip_pooling_max_grad_f32(
    const float* input_data, const float* output_data,
    const float* input_backprop, float* output_backprop,
    const snn_hip_pooling_params* params, int op, void* stream);
/* Average gradient: input_backprop dY [N,OH,OW,C] -> output_backprop dX. */
SNN_HIP_API int snn_hip_pooling_avg_grad_f32(
    const float* input_backprop, float* output_backprop,
    const snn_hip_pooling_params* params, void* stream);
/* The two gradients on half-precision tensors (same operands). */
SNN_HIP_API int snn_hip_pooling_max_grad_f16(
    const void* input_data, const void* output_data,
    const void* input_backprop, void* output_backprop,
    const snn_hip_pooling_params* params, int op, void* stream);
SNN_HIP_API int snn_hip_pooling_avg_grad_f16(
    const void* input_backprop, void* output_backprop,
    const snn_hip_pooling_params* params, void* stream);

/* ---- matmul ----------------------------------------------------------------
 * Stand-in for sycldnn::matmul::internal::launch (src/matmul/launch.cc) as the
 * backend's matmul / batch_matmul members call it
 * (include/portdnn/backend/snn_usm_matmul_provider.h:206-231): row-major
 * C[b] = op(A[b]) * op(B[b]) + beta * C[b], op(A) m x k, op(B) k x n. */
SNN_HIP_API int snn_hip_matmul_f32(const float* lhs, const float* rhs,
                                   float* output, int batches, int m, int k,
                                   int n, int transpose_lhs, int transpose_rhs,
                                   float beta, void* stream);
/* The same on half-precision matrices (products and sums in fp32). */
SNN_HIP_API int snn_hip_matmul_f16(const void* lhs, const void* rhs,
                                   void* output, int batches, int m, int k,
                                   int n, int transpose_lhs, int transpose_rhs,
                                   float beta, void* stream);

/* ---- convolution with bias and activation ---------------------------------
 * No single counterpart in the reference, which runs three launches for this
 * (conv2d::launch, binaryop::launch<Add> with the bias as a [features]
 * operand, pointwise::launch<Relu, Forward>; e.g. the layers of
 * tools/layer.h).  Here the bias add and the activation are folded into the
 * convolution's output stage wherever the chosen kernel writes each output
 * once, and run as one in-place pass otherwise; the result equals the three
 * launches.  `bias` holds one value per feature or is NULL; `activation` is a
 * snn_hip_activation.  Everything else as snn_hip_conv2d_forward_f32. */
typedef enum snn_hip_activation {
  SNN_HIP_ACTIVATION_NONE = 0,
  SNN_HIP_ACTIVATION_RELU = 1
} snn_hip_activation;
SNN_HIP_API int snn_hip_conv2d_forward_bias_act_f32(
    const float* input, const float* filter, const float* bias, float* output,
    const snn_hip_conv2d_params* params, int algorithm, int activation,
    float* workspace, size_t workspace_elems, void* stream);

/* ---- alpha / beta blend ----------------------------------------------------
 * data[i] = alpha * data[i] + beta * prior[i] over n_items elements: the
 * scaling step of the cuDNN-style layer (ScalingParams::applyScaling,
 * include/portdnn/compat/scaling.hpp:150-262, which composes binaryop
 * launches for it).  `prior` may be NULL when beta is 0; a zero alpha drops
 * the data term outright. */
SNN_HIP_API int snn_hip_scale_blend_f32(float* data, const float* prior,
                                        float alpha, float beta,
                                        size_t n_items, void* stream);

/* ---- pointwise -------------------------------------------------------------
 * Stand-ins for sycldnn::pointwise::internal::launch_pointwise
 * (src/pointwise/launch_pointwise_forward.cc, launch_pointwise_grad.cc)
 * reached from sycldnn::pointwise::launch<T, Op, Direction>
 * (include/portdnn/pointwise/launch.h:73-100 forward, :120-150 gradient).
 * `op` is a snn_hip_pointwise_op; n_items must be positive
 * (include/portdnn/internal/pointwise/launch_internal.h:69). */
typedef enum snn_hip_pointwise_op {
  SNN_HIP_POINTWISE_RELU = 0,
  SNN_HIP_POINTWISE_TANH = 1,
  SNN_HIP_POINTWISE_EXP = 2,
  SNN_HIP_POINTWISE_LOG = 3,
  SNN_HIP_POINTWISE_FLOOR = 4,
  SNN_HIP_POINTWISE_SQRT = 5
} snn_hip_pointwise_op;
SNN_HIP_API int snn_hip_pointwise_forward_f32(const float* input, float* output,
                                              size_t n_items, int op,
                                              void* stream);
SNN_HIP_API int snn_hip_pointwise_forward_f16(const void* input, void* output,
                                              size_t n_items, int op,
                                              void* stream);
/* Gradient: input_forward is what the reference's operators call `val` (the
 * forward OUTPUT for relu, tanh, exp and sqrt, the forward INPUT for log;
 * src/pointwise/kernels.h:53-57, :75-77, :100-102, :122-124, :158-160),
 * input_backprop the incoming error.  Floor has no gradient. */
SNN_HIP_API int snn_hip_pointwise_grad_f32(const float* input_forward,
                                           const float* input_backprop,
                                           float* output_backprop,
                                           size_t n_items, int op,
                                           void* stream);
SNN_HIP_API int snn_hip_pointwise_grad_f16(const void* input_forward,
                                           const void* input_backprop,
                                           void* output_backprop,
                                           size_t n_items, int op,
                                           void* stream);

/* ---- binaryop --------------------------------------------------------------
 * Stand-ins for sycldnn::binaryop::internal::launch_binaryop
 * (src/binaryop/launch_binaryop.cc) reached from
 * sycldnn::binaryop::launch<T, Op>
 * (include/portdnn/binaryop/launch.h:61-85).  The dimension lists are
 * BinaryParams::lhs_dims / rhs_dims (include/portdnn/binaryop/params.h:37-46):
 * at most four each (none = scalar), right-aligned, a dimension of 1
 * broadcasts; shapes that do not broadcast return
 * SNN_HIP_INVALID_PARAMETER
 * (include/portdnn/internal/binaryop/launch.h:40-62). */
typedef enum snn_hip_binary_op {
  SNN_HIP_BINARY_ADD = 0,
  SNN_HIP_BINARY_SUB = 1,
  SNN_HIP_BINARY_MUL = 2,
  SNN_HIP_BINARY_DIV = 3
} snn_hip_binary_op;
SNN_HIP_API int snn_hip_binaryop_f32(const float* lhs, const float* rhs,
                                     float* output, const int* lhs_dims,
                                     int n_lhs_dims, const int* rhs_dims,
                                     int n_rhs_dims, int op, void* stream);
SNN_HIP_API int snn_hip_binaryop_f16(const void* lhs, const void* rhs,
                                     void* output, const int* lhs_dims,
                                     int n_lhs_dims, const int* rhs_dims,
                                     int n_rhs_dims, int op, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* SNN_HIP_H_ */
