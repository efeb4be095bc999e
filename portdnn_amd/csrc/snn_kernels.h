// Internal launchers behind the C ABI.  Each returns a snn_hip_status and only
// enqueues work on `stream`.
#ifndef PORTDNN_AMD_CSRC_SNN_KERNELS_H_
#define PORTDNN_AMD_CSRC_SNN_KERNELS_H_

#include "snn_common.h"

namespace snn {

// Algorithm::Direct -- any window / stride, all three directions
// (conv2d_direct.hip).
template <typename T>
int launch_conv2d_direct(int direction, const T* input, const T* filter,
                         T* output, const snn_hip_conv2d_params& p,
                         hipStream_t stream);

// Per-launch options handed down to the kernel launchers.
//  * Work a forward convolution may fold into its last stage: out = act(conv +
//    bias[feature]).  A launcher that applies it sets *applied; otherwise the
//    caller runs launch_bias_act_f32 over the finished output.
//  * deterministic: the launcher must not combine partial sums through float
//    atomics (whose order varies from run to run): no reduction splits.
struct LaunchOptions {
  const float* bias = nullptr;  // one value per feature, or none
  bool relu = false;
  bool* applied = nullptr;
  bool deterministic = false;
  //  * prepare_only: write whatever the launch derives from the filter alone
  //    (the fused Winograd kernels' transformed filter) into the workspace
  //    and launch nothing else; filter_prepared: the workspace already holds
  //    it, from a prepare_only call with the same filter, parameters,
  //    direction and algorithm.  Launchers with nothing to prepare ignore both.
  bool prepare_only = false;
  bool filter_prepared = false;
  bool wanted() const { return bias != nullptr || relu; }
};

// Implicit-GEMM convolution on MFMA (conv2d_igemm.hip): the path behind the
// Tiled and Im2col algorithm tags.  `supports` tells whether the shape meets
// the kernel's vector-width requirements; pointers must be 16-byte aligned.
bool conv2d_igemm_supports(int direction, const snn_hip_conv2d_params& p);
int launch_conv2d_igemm_f32(int direction, const float* input,
                            const float* filter, float* output,
                            const snn_hip_conv2d_params& p, hipStream_t stream,
                            float* workspace = nullptr,
                            size_t workspace_elems = 0,
                            const LaunchOptions* epilogue = nullptr);

// Batched row-major GEMM C[z] = A[z] (m x k) * op(B[z]) on the same MFMA
// kernel, op(B) = B (k x n) or B^T with B stored n x k; operands of
// consecutive problems are contiguous.  `accumulate` adds the product to C
// (float atomics) instead of overwriting it.  `supports` checks k % 32 == 0,
// n % 4 == 0 unless B is transposed, and 16-byte alignment.
bool batched_gemm_mfma_supports(int m, int k, int n, const void* a,
                                const void* b, const void* c,
                                bool transpose_b = false);
int launch_batched_gemm_mfma_f32(const float* a, const float* b, float* c,
                                 int batches, int m, int k, int n,
                                 hipStream_t stream, bool transpose_b = false,
                                 bool accumulate = false,
                                 bool deterministic = false);

// Winograd F(2x2,3x3) convolution, forward and input backprop
// (conv2d_winograd.hip).  `workspace` holds the three transform buffers.
bool conv2d_winograd_supports(int direction, const snn_hip_conv2d_params& p);
int launch_conv2d_winograd_f32(int direction, const float* input,
                               const float* filter, float* output,
                               const snn_hip_conv2d_params& p,
                               float* workspace, size_t workspace_elems,
                               hipStream_t stream, bool deterministic = false);

// One-dimensional Winograd F(2,3) for 1x3 / 3x1 stride-1 windows, forward and
// input backprop (conv2d_winograd_1d.hip).  `..._workspace` is the element
// count needed to run `images` images per pass.
bool conv2d_winograd_1d_supports(int direction, const snn_hip_conv2d_params& p);
size_t conv2d_winograd_1d_workspace(int direction,
                                    const snn_hip_conv2d_params& p, int images);
int launch_conv2d_winograd_1d_f32(int direction, const float* input,
                                  const float* filter, float* output,
                                  const snn_hip_conv2d_params& p,
                                  float* workspace, size_t workspace_elems,
                                  hipStream_t stream,
                                  bool deterministic = false);

// The same convolution in one fused kernel (conv2d_winograd_fused.hip): needs
// channel counts that are multiples of 16 (reduced) and 32 (produced), 16-byte
// aligned pointers and only the transformed-filter part of the workspace.
bool conv2d_winograd_fused_supports(int direction,
                                    const snn_hip_conv2d_params& p);
int launch_conv2d_winograd_fused_f32(int direction, const float* input,
                                     const float* filter, float* output,
                                     const snn_hip_conv2d_params& p,
                                     float* workspace, size_t workspace_elems,
                                     hipStream_t stream,
                                     const LaunchOptions* epilogue = nullptr);

// Winograd F(3x3,2x2) filter gradient of a 3x3 stride-1 convolution in one
// fused kernel (conv2d_winograd_filter.hip).  `workspace` receives one
// partial filter per slice of the tile range; `..._workspace` tells how many
// elements that takes (0 when one work-group per filter block is enough).
bool conv2d_winograd_filter_backprop_supports(const snn_hip_conv2d_params& p);
size_t conv2d_winograd_filter_backprop_workspace(
    const snn_hip_conv2d_params& p);
int launch_conv2d_winograd_filter_backprop_f32(
    const float* x, const float* dy, float* dw, const snn_hip_conv2d_params& p,
    float* workspace, size_t workspace_elems, hipStream_t stream);

// Row-major fp32 GEMM Y = X (m x k) * W (k x n) with the filter in registers
// (gemm_wreg.hip): k = 64, 128, 256 or 512, n in whole feature slices (128 or
// 256 features, or 64 for k <= 256), enough rows to keep 256 persistent
// work-groups busy.  Operands 16-byte aligned.  With `epilogue`, bias (one
// value per column, may be null) is added and relu applied on the way out.
// `transpose_w`: W is stored n x k (the 1x1 input gradient, whose filter
// operand is the HWCF tensor read with the feature index as the reduction).
bool gemm_wreg_supports(int m, int k, int n, bool transpose_w = false);
void launch_gemm_wreg(const float* x, const float* w, float* y, int m, int k,
                      int n, bool epilogue, const float* bias, bool relu,
                      hipStream_t stream, bool transpose_w = false);
// Forward convolution of problems with few output tiles (one 56x56x64 image:
// 49 tiles of 64x64) in one launch without atomics (conv2d_small.hip):
// work-groups of 16 pixels x 64 features whose four waves split the
// reduction.  Channels and features in multiples of 64; 16-byte aligned.
bool conv2d_small_supports(const snn_hip_conv2d_params& p);
int launch_conv2d_small_f32(const float* x, const float* w, float* y,
                            const snn_hip_conv2d_params& p, hipStream_t stream,
                            const LaunchOptions* epilogue = nullptr);
// Stride-1 convolution with windows larger than 1x1 on MFMA with the input
// rows of a run of output pixels resident in LDS (conv2d_rowtile.hip): each
// input element reaches a compute unit once per 64 features instead of once
// per filter tap.  Channels in multiples of 16, features of 64; tensors
// 16-byte aligned.  `transposed_filter`: `filter` is the HWCF tensor of the
// convolution whose input gradient this is (`p` then describes the forward
// convolution over dY: channels and features exchanged, padding window - 1 -
// pad); taps are mirrored and the channel index is the reduction index.
bool conv2d_rowtile_supports(const snn_hip_conv2d_params& p);
int launch_conv2d_rowtile_f32(const float* input, const float* filter,
                              float* output, const snn_hip_conv2d_params& p,
                              hipStream_t stream, bool transposed_filter,
                              const LaunchOptions* epilogue = nullptr);
// The same for deep, small layers (conv2d_rowsplit.hip): every wave of a
// work-group holds all of the tile's 16 x 16 output blocks and one eighth of
// the channels, with its own LDS tile and no barrier in the reduction; the
// eight partial results are added in LDS in a fixed order.  Channels in
// multiples of 128, features of 32; arguments as above.
bool conv2d_rowsplit_supports(const snn_hip_conv2d_params& p);
int launch_conv2d_rowsplit_f32(const float* input, const float* filter,
                               float* output, const snn_hip_conv2d_params& p,
                               hipStream_t stream, bool transposed_filter,
                               const LaunchOptions* epilogue = nullptr);
// Filter gradient with both operands straight from NHWC memory into the fp32
// matrix instruction's registers (conv2d_filter_backprop_direct.hip): a 64 x
// 64 tile of one filter tap of dW per wave, the pixel range split over the
// waves of a work-group (added in LDS) and, for few (tap, tile) units, over
// work-groups, whose partial filters (`partial`, ..._partial_floats(p) floats,
// 16-byte aligned; may be null when that is 0) a second kernel adds in a fixed
// order.  Any window, stride and padding, at least 256 output pixels, all
// pointers 16-byte aligned; channels and features in multiples of 64, or
// (`ragged`) any counts: the tiles that stick out are padded with zeros, and
// counts that are not multiples of 4 are loaded element by element.  The f16
// form reads and writes binary16 tensors, accumulates in fp32 and always goes
// through partial filters (at least one), which the second kernel rounds.
bool conv2d_filter_backprop_direct_f32_supports(const snn_hip_conv2d_params& p,
                                                bool ragged = false);
bool conv2d_filter_backprop_direct_f16_supports(const snn_hip_conv2d_params& p);
// Whether the implicit-GEMM launcher sends this fp32 filter gradient to that
// kernel (conv2d_igemm.hip); `reproducible` keeps shapes here whose faster
// kernel sums through atomics.
bool conv2d_filter_backprop_direct_f32_wanted(const snn_hip_conv2d_params& p,
                                              bool reproducible = false);
size_t conv2d_filter_backprop_direct_f32_partial_floats(
    const snn_hip_conv2d_params& p);
size_t conv2d_filter_backprop_direct_f16_partial_floats(
    const snn_hip_conv2d_params& p);
int launch_conv2d_filter_backprop_direct_f32(const float* input,
                                             const float* output_gradient,
                                             float* filter_gradient,
                                             float* partial,
                                             const snn_hip_conv2d_params& p,
                                             hipStream_t stream);
int launch_conv2d_filter_backprop_direct_f16(const _Float16* input,
                                             const _Float16* output_gradient,
                                             _Float16* filter_gradient,
                                             float* partial,
                                             const snn_hip_conv2d_params& p,
                                             hipStream_t stream);
// Forward convolution of a three-channel image with a 7x7 window, stride 2 and
// 64 features (conv2d_stem.hip): input rows of a band of output rows in LDS,
// the filter in registers.  Output 16-byte aligned, at most 128 output columns.
bool conv2d_stem_supports(const snn_hip_conv2d_params& p);
int launch_conv2d_stem_f32(const float* x, const float* w, float* y,
                           const snn_hip_conv2d_params& p, hipStream_t stream);
// ... and its filter gradient (dw 16-byte aligned; partial filters in a
// stream-ordered temporary).
bool conv2d_stem_input_backprop_supports(const snn_hip_conv2d_params& p);
int launch_conv2d_stem_input_backprop_f32(const float* dy, const float* w,
                                          float* dx,
                                          const snn_hip_conv2d_params& p,
                                          hipStream_t stream);
// (whether that launch adds at most two parts into any dX element, i.e. gives
// the same bits every run)
bool conv2d_stem_input_backprop_reproducible(const snn_hip_conv2d_params& p);
bool conv2d_stem_filter_backprop_supports(const snn_hip_conv2d_params& p);
int launch_conv2d_stem_filter_backprop_f32(const float* x, const float* dy,
                                           float* dw,
                                           const snn_hip_conv2d_params& p,
                                           hipStream_t stream);
// The forward stem kernel with its output -- the large tensor -- rounded to
// binary16 on the store and everything else fp32: what a binary16 stem launch
// runs after widening its image and filter.
int launch_conv2d_stem_f32_to_f16(const float* x, const float* w, _Float16* y,
                                  const snn_hip_conv2d_params& p,
                                  hipStream_t stream);

// The same in half precision with fp32 accumulation (gemm_wreg_f16.hip):
// k = 64, 128, 256 or 512.
bool gemm_wreg_f16_supports(int m, int k, int n);
void launch_gemm_wreg_f16(const _Float16* x, const _Float16* w, _Float16* y,
                          int m, int k, int n, hipStream_t stream);

// Half-precision forward convolution on MFMA (conv2d_igemm_f16.hip).  The
// workspace, when large enough, receives the re-laid-out filter.
bool conv2d_igemm_f16_supports(const snn_hip_conv2d_params& p);
int launch_conv2d_igemm_f16(const _Float16* input, const _Float16* filter,
                            _Float16* output, const snn_hip_conv2d_params& p,
                            _Float16* workspace, size_t workspace_elems,
                            hipStream_t stream);
// Row-major binary16 GEMM y[m][n] = sum_k x[m][k] w[k][n] with the filter slab
// resident in LDS (gemm_rows_f16.hip): 1x1 stride-1 convolutions and matmul
// with k a multiple of 64 and n a multiple of 64; needs no workspace.
bool gemm_rows_f16_supports(int m, int k, int n);
int launch_gemm_rows_f16(const _Float16* x, const _Float16* w, _Float16* y,
                         int m, int k, int n, hipStream_t stream);
// Halves of caller workspace the half-precision forward and input-gradient
// launchers use for the re-laid-out filter (0: none needed).
size_t conv2d_f16_filter_pack_halves(int direction,
                                     const snn_hip_conv2d_params& p);
// Stride-1 input gradient in half precision: the forward kernels above run on
// dY with the filter's taps mirrored and its channel / feature roles swapped.
// `supports` is false when neither kernel takes the shape.
bool conv2d_input_backprop_f16_supports(const snn_hip_conv2d_params& p);
int launch_conv2d_input_backprop_f16(const _Float16* dy,
                                     const _Float16* filter, _Float16* dx,
                                     const snn_hip_conv2d_params& p,
                                     _Float16* workspace,
                                     size_t workspace_elems,
                                     hipStream_t stream);

// Half-precision strided input gradient by stride classes (conv2d_igemm.hip):
// every class of input pixels modulo the strides is a dense stride-1 forward
// convolution of dY on the binary16 kernels.  Features in multiples of 64,
// channels of 4, from 2^30 multiply-adds; the launch returns -1 when the
// geometry does not fit (then nothing was launched).
bool conv2d_strided_input_backprop_f16_supports(const snn_hip_conv2d_params& p);
int launch_conv2d_strided_input_backprop_f16(const _Float16* output_gradient,
                                             const _Float16* filter,
                                             _Float16* input_gradient,
                                             const snn_hip_conv2d_params& p,
                                             hipStream_t stream);

// Half-precision forward convolution for the shapes the binary16 kernels do
// not take (conv2d_igemm.hip): the general implicit-GEMM kernel reading
// binary16 operands.  Channels and features in multiples of 4.
bool conv2d_forward_general_f16_supports(const snn_hip_conv2d_params& p);
int launch_conv2d_forward_general_f16(const _Float16* input,
                                      const _Float16* filter, _Float16* output,
                                      const snn_hip_conv2d_params& p,
                                      hipStream_t stream);

// Half-precision gradients on the fp32 matrix instructions
// (conv2d_igemm.hip): the filter gradient for channel counts in multiples of
// 64 (fp32 accumulation buffer in the workspace when it holds twice the
// filter's element count, else a stream-ordered temporary), and the input
// gradient for the shapes launch_conv2d_input_backprop_f16 does not take.
// conv2d_filter_backprop_f16.hip: 3x3 stride-1 SAME filter gradient on the
// binary16 matrix cores (channels and features multiples of 64).  `part` is
// scratch of ..._partial_floats(p) floats for the partial tiles.
bool conv2d_filter_backprop_3x3_f16_supports(const snn_hip_conv2d_params& p);
size_t conv2d_filter_backprop_3x3_f16_partial_floats(
    const snn_hip_conv2d_params& p);
int launch_conv2d_filter_backprop_3x3_f16(const _Float16* x,
                                          const _Float16* dy, _Float16* dw,
                                          float* part,
                                          const snn_hip_conv2d_params& p,
                                          hipStream_t stream);
// The same for 1x1 stride-1 unpadded layers (one flat stream of pixels).
bool conv2d_filter_backprop_1x1_f16_supports(const snn_hip_conv2d_params& p);
size_t conv2d_filter_backprop_1x1_f16_partial_floats(
    const snn_hip_conv2d_params& p);
int launch_conv2d_filter_backprop_1x1_f16(const _Float16* x,
                                          const _Float16* dy, _Float16* dw,
                                          float* part,
                                          const snn_hip_conv2d_params& p,
                                          hipStream_t stream);
bool conv2d_filter_backprop_f16_supports(const snn_hip_conv2d_params& p);
int launch_conv2d_filter_backprop_f16(const _Float16* x, const _Float16* dy,
                                      _Float16* dw,
                                      const snn_hip_conv2d_params& p,
                                      _Float16* workspace,
                                      size_t workspace_elems,
                                      hipStream_t stream);
bool conv2d_input_backprop_general_f16_supports(
    const snn_hip_conv2d_params& p);
int launch_conv2d_input_backprop_general_f16(const _Float16* dy,
                                             const _Float16* filter,
                                             _Float16* dx,
                                             const snn_hip_conv2d_params& p,
                                             hipStream_t stream);

// Half-precision stride-1 forward convolution with the input tile resident
// in LDS (conv2d_rowtile_f16.hip).  `packed` receives the filter in MFMA
// operand order: window_rows * window_cols * channels * features halves,
// 16-byte aligned.  With `transposed_filter` the filter is read as the input
// gradient's: `p` then describes the gradient as a forward convolution of dY
// (channels = the original features and vice versa, padding window - 1 - pad)
// and `filter` is still the original HWCF tensor.
bool conv2d_rowtile_f16_supports(const snn_hip_conv2d_params& p);
int launch_conv2d_rowtile_f16(const _Float16* input, const _Float16* filter,
                              _Float16* output, const snn_hip_conv2d_params& p,
                              _Float16* packed, hipStream_t stream,
                              bool transposed_filter = false);

// Depthwise convolution, all three directions (depthwise.hip).  With
// `static_scratch` (the library's own scratch array) the filter gradient
// takes its partial-filter buffer from there and allocates nothing.
template <typename T>
int launch_depthwise(int direction, const T* input, const T* filter, T* output,
                     const snn_hip_depthwise_params& p, hipStream_t stream,
                     float* static_scratch = nullptr);
// The fp32 filter gradient with the partial filters in the library's
// file-scope device array: no allocation of any kind.
int launch_depthwise_filter_backprop_noalloc_f32(
    const float* input, const float* dy, float* dw,
    const snn_hip_depthwise_params& p, hipStream_t stream);

// Pooling (pooling.hip).
template <typename T>
int launch_pooling_forward(const T* input, T* output,
                           const snn_hip_pooling_params& p, int op,
                           hipStream_t stream);
int launch_pooling_max_grad(const float* input_data, const float* output_data,
                            const float* input_backprop,
                            float* output_backprop,
                            const snn_hip_pooling_params& p, int op,
                            hipStream_t stream);
int launch_pooling_avg_grad(const float* input_backprop,
                            float* output_backprop,
                            const snn_hip_pooling_params& p,
                            hipStream_t stream);
int launch_pooling_max_grad_f16(const _Float16* input_data,
                                const _Float16* output_data,
                                const _Float16* input_backprop,
                                _Float16* output_backprop,
                                const snn_hip_pooling_params& p, int op,
                                hipStream_t stream);
int launch_pooling_avg_grad_f16(const _Float16* input_backprop,
                                _Float16* output_backprop,
                                const snn_hip_pooling_params& p,
                                hipStream_t stream);

// Batched row-major GEMM on MFMA (matmul.hip).
int launch_matmul_f32(const float* lhs, const float* rhs, float* output,
                      int batches, int m, int k, int n, bool transpose_lhs,
                      bool transpose_rhs, float beta, hipStream_t stream);
int launch_matmul_f16(const _Float16* lhs, const _Float16* rhs,
                      _Float16* output, int batches, int m, int k, int n,
                      bool transpose_lhs, bool transpose_rhs, float beta,
                      hipStream_t stream);

// Element-wise operators (elementwise.hip).  `op` is a snn_hip_pointwise_op
// or snn_hip_binary_op; operands may alias the output element for element.
int launch_pointwise_forward_f32(int op, const float* in, float* out, size_t n,
                                 hipStream_t stream);
int launch_pointwise_forward_f16(int op, const _Float16* in, _Float16* out,
                                 size_t n, hipStream_t stream);
int launch_pointwise_grad_f32(int op, const float* val, const float* err,
                              float* out, size_t n, hipStream_t stream);
int launch_pointwise_grad_f16(int op, const _Float16* val, const _Float16* err,
                              _Float16* out, size_t n, hipStream_t stream);
int launch_binaryop_f32(int op, const float* lhs, const float* rhs, float* out,
                        const int* lhs_dims, int n_lhs, const int* rhs_dims,
                        int n_rhs, hipStream_t stream);
int launch_binaryop_f16(int op, const _Float16* lhs, const _Float16* rhs,
                        _Float16* out, const int* lhs_dims, int n_lhs,
                        const int* rhs_dims, int n_rhs, hipStream_t stream);
// data[i] = act(data[i] + bias[i % features]) in place over n elements
// (n % features == 0); bias may be null, act is max(., 0) when relu.
int launch_bias_act_f32(float* data, const float* bias, int features, size_t n,
                        bool relu, hipStream_t stream);
// data[i] = alpha * data[i] + beta * prior[i] (prior may be null when beta is
// 0): the blend of the compatibility layer's alpha / beta scaling.
int launch_scale_blend_f32(float* data, const float* prior, float alpha,
                           float beta, size_t n, hipStream_t stream);

// Layout conversions (layout.hip).  out[b][c][r] = in[b][r][c] for every
// batch b (NCHW -> NHWC with rows = C, cols = H * W, and back with the two
// swapped); FCHW <-> HWCF filters with taps = R * S.
int launch_transpose_batched_f32(const float* in, float* out, int batches,
                                 int rows, int cols, hipStream_t stream);
int launch_permute_filter_f32(const float* in, float* out, int features,
                              int channels, int taps, bool to_hwcf,
                              hipStream_t stream);

}  // namespace snn

#endif  // PORTDNN_AMD_CSRC_SNN_KERNELS_H_
