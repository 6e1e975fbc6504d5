/*
 * C ABI of libptl_hip.so: the matmul-based training core of PULP-TrainLib
 * (Conv2D / pointwise / depthwise / Linear, forward + weight-gradient +
 * input-gradient, fp32 and IEEE fp16) running as HIP kernels on gfx950.
 *
 * Part 1 are the reference's own entry points: same names, same
 * `void f(void *args)` signature, same argument structs (ptl_structs.h).
 * Part 2 are the extensions a GPU needs and the reference has no word for:
 * batched calls, stream/timing control, error reporting.
 *
 * Pointers inside the argument structs may be host or device pointers; the
 * kind is detected per pointer.  Device pointers are used in place and the
 * call returns after enqueueing on the library stream (ptl_sync() waits).
 * Host pointers are staged through temporary device buffers and the call
 * returns with the results already copied back.
 *
 * Semantics where the reference is not self-consistent (padding on the
 * im2col weight/input-gradient path, pointwise input gradient with
 * Cin != Cout, pad_tensor with pads other than 1): the textbook operation,
 * i.e. what the reference's naive kernels compute.  matmul_type ids are
 * accepted and validated but all select the same MFMA kernel family: every
 * reference variant computes the same product.
 */
#ifndef PTL_API_H
#define PTL_API_H

#include "ptl_structs.h"

#ifdef __cplusplus
extern "C" {
#endif

/* ------------------------------------------------------------------ */
/* Part 1: reference entry points                                      */
/* ------------------------------------------------------------------ */

/* Conv2D, fp32: lib/sources/pulp_conv2d_fp32.c:27, :225, :240, :454 */
void pulp_conv2d_fp32_fw_cl(void *Conv2D_args);
void pulp_conv2d_fp32_bw_cl(void *Conv2D_args);
void pulp_conv2d_fp32_bw_param_grads_cl(void *Conv2D_args);
void pulp_conv2d_fp32_bw_input_grads_cl(void *Conv2D_args);
/* Conv2D, fp16: lib/sources/pulp_conv2d_fp16.c:27, :225, :240, :454 */
void pulp_conv2d_fp16_fw_cl(void *Conv2D_args_fp16);
void pulp_conv2d_fp16_bw_cl(void *Conv2D_args_fp16);
void pulp_conv2d_fp16_bw_param_grads_cl(void *Conv2D_args_fp16);
void pulp_conv2d_fp16_bw_input_grads_cl(void *Conv2D_args_fp16);

/* Pointwise conv: lib/sources/pulp_conv_pw_fp32.c:27, :106, :121, :233 */
void pulp_conv_pw_fp32_fw_cl(void *PointWise_Conv_args);
void pulp_conv_pw_fp32_bw_cl(void *PointWise_Conv_args);
void pulp_conv_pw_fp32_bw_param_grads_cl(void *PointWise_Conv_args);
void pulp_conv_pw_fp32_bw_input_grads_cl(void *PointWise_Conv_args);
/* lib/sources/pulp_conv_pw_fp16.c:27, :108, :123, :249 */
void pulp_conv_pw_fp16_fw_cl(void *PointWise_Conv_args_fp16);
void pulp_conv_pw_fp16_bw_cl(void *PointWise_Conv_args_fp16);
void pulp_conv_pw_fp16_bw_param_grads_cl(void *PointWise_Conv_args_fp16);
void pulp_conv_pw_fp16_bw_input_grads_cl(void *PointWise_Conv_args_fp16);

/* Depthwise conv: lib/sources/pulp_conv_dw_fp32.c:27, :49, :65, :77 */
void pulp_conv_dw_fp32_fw_cl(void *DepthWise_Conv_args);
void pulp_conv_dw_fp32_bw_cl(void *DepthWise_Conv_args);
void pulp_conv_dw_fp32_bw_param_grads_cl(void *DepthWise_Conv_args);
void pulp_conv_dw_fp32_bw_input_grads_cl(void *DepthWise_Conv_args);
/* lib/sources/pulp_conv_dw_fp16.c:28, :44, :61, :75 */
void pulp_conv_dw_fp16_fw_cl(void *DepthWise_Conv_args_fp16);
void pulp_conv_dw_fp16_bw_cl(void *DepthWise_Conv_args_fp16);
void pulp_conv_dw_fp16_bw_param_grads_cl(void *DepthWise_Conv_args_fp16);
void pulp_conv_dw_fp16_bw_input_grads_cl(void *DepthWise_Conv_args_fp16);

/* Linear: lib/sources/pulp_linear_fp32.c:25, :67, :85, :142 */
void pulp_linear_fp32_fw_cl(void *Linear_args);
void pulp_linear_fp32_bw_cl(void *Linear_args);
void pulp_linear_fp32_bw_param_grads_cl(void *Linear_args);
void pulp_linear_fp32_bw_input_grads_cl(void *Linear_args);
/* lib/sources/pulp_linear_fp16.c:25, :72, :90, :149 */
void pulp_linear_fp16_fw_cl(void *Linear_args_fp16);
void pulp_linear_fp16_bw_cl(void *Linear_args_fp16);
void pulp_linear_fp16_bw_param_grads_cl(void *Linear_args_fp16);
void pulp_linear_fp16_bw_input_grads_cl(void *Linear_args_fp16);

/* Multi-head self-attention training step, fp32: lib/sources/pulp_mhsa_fp32.c:20 (forward), :648 (backward).
 * Forward fills q, k, v, softmax_buffer, attention_map and output; backward reads them and fills every
 * `diff` (input->diff is added to, as the reference's closing vector sums do, :1634-1745).
 * Softmax uses the reference's approximate exponential (fastexp_gist, lib/sources/pulp_train_utils_fp32.c:1223)
 * and the projection biases are per feature (row of the F x L matrices). */
void pulp_mhsa_fp32_fw_cl(void *Mhsa_args);
void pulp_mhsa_fp32_bw_cl(void *Mhsa_args);
/* Row-wise softmax with the approximate exponential and its backward pass:
 * lib/sources/pulp_act_fp32.c:187, :335. */
void pulp_softmax_fp32_fw_cl(void *softmax_args);
void pulp_softmax_fp32_bw_cl(void *softmax_args);

/* Layers around the matmul core in a ResNet-style step.
 * ReLU: lib/sources/pulp_act_fp32.c:83-129, pulp_act_fp16.c (same structure). */
void pulp_relu_fp32_fw_cl(void *act_args);
void pulp_relu_fp32_bw_cl(void *act_args);
void relu_core_fw_fp32(void *act_args);
void relu_core_bw_fp32(void *act_args);
void pulp_relu_fp16_fw_cl(void *act_args_fp16);
void pulp_relu_fp16_bw_cl(void *act_args_fp16);
void relu_core_fw_fp16(void *act_args_fp16);
void relu_core_bw_fp16(void *act_args_fp16);
/* Residual connection: lib/sources/pulp_residual_fp32.c:26 (output = skip + lout), :59 (skip->diff +=
 * output->diff unless skip_in_grad), :92 (lout->diff = output->diff); pulp_residual_fp16.c:30, :67, :100. */
void pulp_residualconn_fp32_fw(void *SkipConn_args);
void pulp_sumnode_fp32_bw(void *SkipConn_args);
void pulp_residualconn_fp32_bw(void *SkipConn_args);
void pulp_residualconn_fp16_fw(void *SkipConn_args_fp16);
void pulp_sumnode_fp16_bw(void *SkipConn_args_fp16);
void pulp_residualconn_fp16_bw(void *SkipConn_args_fp16);
/* Average pooling: lib/sources/pulp_pooling_fp32.c:24, :69; pulp_pooling_fp16.c:24, :69. */
void pulp_avgpool_fp32_fw_cl(void *pool_args);
void pulp_avgpool_fp32_bw_cl(void *pool_args);
void pulp_avgpool_fp16_fw_cl(void *pool_args_fp16);
void pulp_avgpool_fp16_bw_cl(void *pool_args_fp16);
/* Cross-entropy over raw logits: lib/sources/pulp_losses_fp32.c:26, :91; pulp_losses_fp16.c:26, :88. */
void pulp_CrossEntropyLoss(void *loss_args);
void pulp_CrossEntropyLoss_backward(void *loss_args);
void pulp_CrossEntropyLoss_fp16(void *loss_args_fp16);
void pulp_CrossEntropyLoss_backward_fp16(void *loss_args_fp16);
/* Gradient descent with optional weight decay: lib/sources/pulp_optimizers_fp32.c:26, pulp_optimizers_fp16.c:26. */
void pulp_gradient_descent_fp32(void *optim_args);
void pulp_gradient_descent_fp16(void *optim_args_fp16);
/* Batch normalisation forward: lib/sources/pulp_batchnorm_fp32.c:28-114 (the reference has no backward). */
void pulp_batch_norm_fp32_fw_cl(void *BatchNorm_args_fp32);
void pulp_batch_norm_parallelized_fp32_fw_cl(void *BatchNorm_args_fp32);

/* Matmul kernels and their dispatcher.
 * mm / mm_M: lib/sources/pulp_matmul_fp32.c:190, :345
 * mm_fp16 / mm_M_fp16: lib/sources/pulp_matmul_fp16.c:191, :273
 * mm_manager: lib/sources/pulp_train_utils_fp32.c:1330 (ids 0..23)
 * mm_manager_fp16: lib/sources/pulp_train_utils_fp16.c:1258 (ids 0..8) */
void mm(void *matMul_args);
void mm_M(void *matMul_args);
void mm_fp16(void *matMul_args_fp16);
void mm_M_fp16(void *matMul_args_fp16);
/* The unrolled variants, by name (lib/include/pulp_matmul_fp32.h:72-244; lib/include/pulp_matmul_fp16.h:56-107):
 * each computes the product of mm / mm_fp16; the reference's matmul harness calls them by name
 * (tests/test_matmul/net.c:95-186). */
void mm_u2(void *matMul_args);
void mm_unroll_1x2(void *matMul_args);
void mm_unroll_1x4(void *matMul_args);
void mm_unroll_1x8(void *matMul_args);
void mm_unroll_2x1(void *matMul_args);
void mm_unroll_4x1(void *matMul_args);
void mm_unroll_8x1(void *matMul_args);
void mm_unroll_2x2(void *matMul_args);
void mm_unroll_2x4(void *matMul_args);
void mm_unroll_4x2(void *matMul_args);
void mm_unroll_4x4(void *matMul_args);
void mm_M_u2(void *matMul_args);
void mm_M_unroll_2x1(void *matMul_args);
void mm_M_unroll_4x1(void *matMul_args);
void mm_M_unroll_8x1(void *matMul_args);
void mm_M_unroll_1x2(void *matMul_args);
void mm_M_unroll_1x4(void *matMul_args);
void mm_M_unroll_1x8(void *matMul_args);
void mm_M_unroll_2x2(void *matMul_args);
void mm_M_unroll_4x2(void *matMul_args);
void mm_M_unroll_2x4(void *matMul_args);
void mm_M_unroll_4x4(void *matMul_args);
void mm_fp16_SIMD_2x4(void *matMul_args_fp16);
void mm_fp16_SIMD_4x8(void *matMul_args_fp16);
void mm_fp16_unroll_8x1(void *matMul_args_fp16);
void mm_fp16_unroll_4x1(void *matMul_args_fp16);
void mm_fp16_unroll_2x1(void *matMul_args_fp16);
void mm_M_fp16_SIMD_2x4(void *matMul_args_fp16);
void mm_M_fp16_SIMD_4x8(void *matMul_args_fp16);
/* Matrix x vector, C[i] = sum_k A[i*K+k] * B[k] (lib/include/pulp_matmul_fp16.h:118-135;
 * lib/sources/pulp_matmul_fp16.c:1158): with M > 1 and trans_B set, M is the vector's length; with M > 1 and
 * trans_B clear the reference stops the program, this library prints the same message and rejects the call. */
void mv_fp16_SIMD_2x1(void *matMul_args_fp16);
void mv_fp16_SIMD_4x1(void *matMul_args_fp16);
void mv_fp16_SIMD_8x1(void *matMul_args_fp16);
void mm_manager(void *mm_manager_args);
void mm_manager_fp16(void *mm_manager_args_fp16);

/* Kernels forked by the layer entry points in the reference; exported so
 * that code which forks them directly keeps linking.
 * lib/sources/pulp_conv2d_fp32.c:669, :746; pulp_linear_fp32.c:199, :234 */
void im2col_conv2d_fw_kernel(void *mm_manager_args);
void im2col_conv2d_param_grad_kernel(void *mm_manager_args);
void pulp_linear_fp32_fw_cl_kernel(void *mm_manager_args);
void pulp_linear_fp32_bw_param_grads_cl_kernel(void *mm_manager_args);

/* Direct (naive) convolution kernels on matMul_args, textbook stride/pad:
 * lib/sources/pulp_conv_naive_fp32.c:198, :302, :410; _fp16.c twins. */
void naive_conv2d_fw_kernel_CHW(void *matMul_args);
void naive_conv2d_param_grad_kernel_CHW(void *matMul_args);
void naive_conv2d_in_grad_kernel_CHW(void *matMul_args);
void naive_conv2d_fw_kernel_CHW_fp16(void *matMul_args_fp16);
void naive_conv2d_param_grad_kernel_CHW_fp16(void *matMul_args_fp16);
void naive_conv2d_in_grad_kernel_CHW_fp16(void *matMul_args_fp16);

/* The same kernels with the geometry fixed by the name: 3x3 or 5x5 filter, stride 2, padding 1 on every side
 * (only H, W, pCin, pCout, the pointers and the bias fields of the struct are read):
 * lib/sources/pulp_conv_naive_fp32.c:520, :581, :643, :702, :762, :825;
 * lib/sources/pulp_conv_naive_fp16.c:471, :529, :588, :645, :703, :756. */
void naive_conv2d_fw_kernel_CHW_k3x3_s2_p1(void *matMul_args);
void naive_conv2d_param_grad_kernel_CHW_k3x3_s2_p1(void *matMul_args);
void naive_conv2d_in_grad_kernel_CHW_k3x3_s2_p1(void *matMul_args);
void naive_conv2d_fw_kernel_CHW_k5x5_s2_p1(void *matMul_args);
void naive_conv2d_param_grad_kernel_CHW_k5x5_s2_p1(void *matMul_args);
void naive_conv2d_in_grad_kernel_CHW_k5x5_s2_p1(void *matMul_args);
void naive_conv2d_fw_kernel_CHW_k3x3_s2_p1_fp16(void *matMul_args_fp16);
void naive_conv2d_param_grad_kernel_CHW_k3x3_s2_p1_fp16(void *matMul_args_fp16);
void naive_conv2d_in_grad_kernel_CHW_k3x3_s2_p1_fp16(void *matMul_args_fp16);
void naive_conv2d_fw_kernel_CHW_k5x5_s2_p1_fp16(void *matMul_args_fp16);
void naive_conv2d_param_grad_kernel_CHW_k5x5_s2_p1_fp16(void *matMul_args_fp16);
void naive_conv2d_in_grad_kernel_CHW_k5x5_s2_p1_fp16(void *matMul_args_fp16);

/* Bias add on a row-major H x W matrix (t == 0: bias[column], else bias[row]), the epilogue mm_manager runs
 * when USE_BIASES == 1: lib/sources/pulp_train_utils_fp32.c:1286, lib/include/pulp_train_utils_fp16.h:783. */
void mm_bias_add_transposed(void *mm_bias_add_args);
void mm_bias_add_transposed_fp16(void *mm_bias_add_args_fp16);

/* Depthwise kernels: lib/sources/pulp_conv_naive_fp32.c:29, :113, :153;
 * lib/sources/pulp_conv_naive_fp16.c:32, :75, :118 */
void dw_kernel_forward(void *kernel_DW_args);
void dw_kernel_weight_grad(void *kernel_DW_args);
void dw_kernel_input_grad(void *kernel_DW_args);
void dw_kernel_forward_fp16(void *kernel_DW_args_fp16);
void dw_kernel_weight_grad_fp16(void *kernel_DW_args_fp16);
void dw_kernel_input_grad_fp16(void *kernel_DW_args_fp16);

/* Materialising patch-matrix builders and the weight block transpose
 * (index work, bit-exact): lib/sources/pulp_im2col_fp32.c:29, :668, :1020;
 * lib/sources/pulp_im2col_fp16.c:29, :526, :882.  The layer entry points
 * above do not call these (their im2col is implicit); they exist for
 * callers that use the buffers themselves. */
void pulp_im2row_fp32(void *im2col_args);
void pulp_im2col_fp32(void *im2col_args);
void pulp_blocktransp_fp32(void *blocktransp_args);
void pulp_im2row_fp16(void *im2col_args_fp16);
void pulp_im2col_fp16(void *im2col_args_fp16);
void pulp_blocktransp_fp16(void *blocktransp_args_fp16);

/* Layout / transposition / streaming helpers:
 * lib/sources/pulp_train_utils_fp32.c:39 (transpose_matrix), :79 (transpose),
 * :186 (copy), :197 (set_to_value), :208 (vect_sum), :809 (cast), :821
 * (HWC_to_CHW), :875 (CHW_to_HWC), :929 (pad_tensor); fp16 twins in
 * lib/sources/pulp_train_utils_fp16.c:40-1000. */
void transpose_matrix(void *transp_args);
void transpose(void *transp_args);
void copy(void *copy_args);
void set_to_value(void *set_to_value_args);
void vect_sum(void *vect_sum_args);
void cast_fp16_tensor_to_fp32(void *cast_16t32_args);
void HWC_to_CHW(void *layout_args);
void CHW_to_HWC(void *layout_args);
void pad_tensor(void *pad_args);
void transpose_matrix_fp16(void *transp_args_fp16);
void transpose_fp16(void *transp_args_fp16);
void copy_fp16(void *copy_args_fp16);
void set_to_value_fp16(void *set_to_value_args_fp16);
void vect_sum_fp16(void *vect_sum_args_fp16);
void cast_fp32_tensor_to_fp16(void *cast_32t16_args);
void HWC_to_CHW_fp16(void *layout_args_fp16);
void CHW_to_HWC_fp16(void *layout_args_fp16);
void pad_tensor_fp16(void *pad_args_fp16);

/* ------------------------------------------------------------------ */
/* Part 2: extensions (no counterpart in the reference)                */
/* ------------------------------------------------------------------ */

/* Select the device and create the library state.  Returns 0 on success.
 * Every other call initialises lazily on the current device if needed, and
 * fails (non-zero, message in ptl_last_error) when no HIP device exists:
 * there is no CPU fallback. */
int ptl_init(int device);
/* Message of the last failed call on this thread ("" if none). */
const char *ptl_last_error(void);
/* Status of the last reference-style (void) entry point on this thread:
 * 0 = ran, 1 = rejected its arguments (message printed, outputs untouched),
 * 2 = a HIP call failed. */
int ptl_last_status(void);
/* Stream on which kernels are enqueued (a hipStream_t); NULL = default.  The stream being left is drained first
 * (its kernels may still use the library's buffers).  Must not be called while that stream is being captured into
 * a graph: the call is then refused (ptl_last_status() == 1, the stream stays); a drain that fails is reported
 * with status 2 after the switch. */
void ptl_set_stream(void *hip_stream);
/* The library keeps two internal device buffers (partial sums of split contractions; blocked / padded / dilated
 * copies) that grow when a call needs more - by synchronising the device, freeing and allocating, which is illegal
 * while a stream is being captured and unwelcome in a steady-state loop.  ptl_reserve grows them to at least the
 * given sizes now (0 = leave); ptl_reserved reports their present sizes, so a caller can run its shapes once,
 * read the sizes and reserve them at start-up the next time.  A call that would have to grow a buffer while the
 * library's stream is being captured fails with status 2 and an error text that names ptl_reserve, and the
 * capture stays valid.  No counterpart in the reference (its callers own every buffer). */
int ptl_reserve(size_t workspace_bytes, size_t scratch_bytes);
void ptl_reserved(size_t *workspace_bytes, size_t *scratch_bytes);
int ptl_sync(void);
/* Kernel selection: 0 (default) = the fastest kernel that fits the problem
 * (direct convolution for large channel-major Conv2D forward / input-gradient
 * calls, the LDS-DMA pipelined GEMM elsewhere, the register-staged GEMM as the
 * last resort); 1 = the register-staged GEMM only; 2 = as 0, but the direct
 * convolution kernel is taken whenever the geometry fits it, however small the
 * call; 3 = as 0, but the sum-over-filter-taps route (unit-stride layers whose
 * channel counts fill whole 128-byte slabs) is taken whenever the geometry fits
 * it, on the pipelined GEMM; 5 = the same route with the input tile resident in
 * LDS for all taps (3x3 unit-stride fp16 layers with channel counts in multiples
 * of 64: channel-major on a prepared copy of the input, channel-minor "same"
 * layers on the caller's tensors in place) wherever that kernel fits;
 * 6 = as 0, but the kernels for small channel-major layers (3x3 or 1x1 filters,
 * stride 1 or 2, at most 64 channels on either side, fp16 and fp32; by default
 * only up to four - for layers narrower than 64 channels sixteen - workgroups
 * per compute unit, and for the weight gradient only up to 262144 positions)
 * are taken whenever the geometry fits them.
 * All routes compute the same products.
 * ptl_last_conv_direct() tells whether the last Conv2D call ran one of the
 * convolution kernels (1) or the implicit-im2col GEMM (0);
 * ptl_last_gemm_streamed() whether the last product that went to the pipelined
 * GEMM ran its streaming kernel (resident row panel, column tiles streamed:
 * the route of pointwise layers over a batch) (1) or a tile-per-workgroup
 * kernel (0); ptl_last_conv_resident() whether the last Conv2D call that took
 * the tap route kept its input tile in LDS (1), or ran the small-layer kernels
 * (2: forward, either gradient, or both gradients in one call; 3: the forward
 * kernel that also applied the normalisation in front of the layer, see
 * ptl_conv2d_*_fw_batched_normed);
 * ptl_last_gemm_tile() the output tile of the last product that ran a tile-per-workgroup kernel of the
 * look-up-free pipelined GEMM, as rows * 1000 + columns (256256 = 256 x 256, 128064 = 128 x 64). */
void ptl_set_gemm_path(int path);
int ptl_last_conv_direct(void);
int ptl_last_gemm_streamed(void);
int ptl_last_conv_resident(void);
int ptl_last_gemm_tile(void);
/* A measurement aid (no counterpart in the reference, not on the training path): the rate, in TFLOP/s, that this
 * board sustains on a loop of nothing but fp16 MFMAs - shape 32: v_mfma_f32_32x32x16_f16, 16: v_mfma_f32_16x16x32_f16 -
 * on random (1) or all-zero (0) operands, with one or two waves per SIMD on every compute unit, `iters` x 262144 flops
 * per wave.  On random operands such a loop runs against the board's power limit; the rate it holds is what a GEMM
 * or convolution kernel can approach on that data.  Uses the library's scratch buffer and event pair. */
int ptl_probe_mfma_fp16(int shape, int random_operands, int waves_per_simd, int iters, float *tflops);
/* hipEvent timing on the library stream: begin records, end records,
 * synchronises and returns the elapsed milliseconds (negative on error). */
int ptl_timer_begin(void);
float ptl_timer_end_ms(void);

/* Batched mode: `nsamples` independent samples stored back to back.
 * input/output blobs describe ONE sample (C,H,W,dim); sample n of a blob
 * lives at data + n*dim (diff + n*dim).  Forward and input-gradient
 * results are per sample; the weight gradient written to coeff->diff is
 * the SUM over the samples (overwriting, like the reference's single-sample
 * call).  nsamples = 1 is exactly the reference entry point.  Return 0 on
 * success, non-zero after rejecting the arguments or a HIP failure. */
int ptl_conv2d_fp32_fw_batched(const struct Conv2D_args *a, int nsamples);
int ptl_conv2d_fp32_wg_batched(const struct Conv2D_args *a, int nsamples);
int ptl_conv2d_fp32_ig_batched(const struct Conv2D_args *a, int nsamples);
int ptl_conv2d_fp16_fw_batched(const struct Conv2D_args_fp16 *a, int nsamples);
int ptl_conv2d_fp16_wg_batched(const struct Conv2D_args_fp16 *a, int nsamples);
int ptl_conv2d_fp16_ig_batched(const struct Conv2D_args_fp16 *a, int nsamples);

int ptl_conv_pw_fp32_fw_batched(const struct PointWise_Conv_args *a, int nsamples);
int ptl_conv_pw_fp32_wg_batched(const struct PointWise_Conv_args *a, int nsamples);
int ptl_conv_pw_fp32_ig_batched(const struct PointWise_Conv_args *a, int nsamples);
int ptl_conv_pw_fp16_fw_batched(const struct PointWise_Conv_args_fp16 *a, int nsamples);
int ptl_conv_pw_fp16_wg_batched(const struct PointWise_Conv_args_fp16 *a, int nsamples);
int ptl_conv_pw_fp16_ig_batched(const struct PointWise_Conv_args_fp16 *a, int nsamples);

int ptl_conv_dw_fp32_fw_batched(const struct DepthWise_Conv_args *a, int nsamples);
int ptl_conv_dw_fp32_wg_batched(const struct DepthWise_Conv_args *a, int nsamples);
int ptl_conv_dw_fp32_ig_batched(const struct DepthWise_Conv_args *a, int nsamples);
int ptl_conv_dw_fp16_fw_batched(const struct DepthWise_Conv_args_fp16 *a, int nsamples);
int ptl_conv_dw_fp16_wg_batched(const struct DepthWise_Conv_args_fp16 *a, int nsamples);
int ptl_conv_dw_fp16_ig_batched(const struct DepthWise_Conv_args_fp16 *a, int nsamples);

/* No counterpart in the reference: ptl_conv_dw_fp16_wg_batched for callers that cannot allocate device
 * memory (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  Same
 * arguments, same kernels, same result; the partial sums live in a fixed 1 MiB device array that every call on
 * a GPU shares (calls that overlap on one GPU race; nothing in it needs clearing between calls).  Every tensor
 * pointer must be a device pointer, ptl_init() must have run, and a call whose partial sums would not fit
 * (more than 1 MiB: C x sample groups x taps floats, e.g. 64 x 16 x 9) is rejected with status 1.  Calls no
 * hipMalloc / hipFree. */
int ptl_conv_dw_fp16_wg_noalloc(const struct DepthWise_Conv_args_fp16 *a, int nsamples);

/* Weight and input gradient of a Conv2D batch in ONE call, as pulp_conv2d_fp32_bw_cl / pulp_conv2d_fp16_bw_cl do
 * for one sample (lib/sources/pulp_conv2d_fp32.c:225-237, lib/sources/pulp_conv2d_fp16.c:225); honours skip_wg_grad /
 * skip_in_grad.  fp16 channel-major 3x3 "same" layers that run the resident-tile kernels share one channel-blocked
 * copy of the output gradient between the two steps. */
int ptl_conv2d_fp32_bw_batched(const struct Conv2D_args *a, int nsamples);
int ptl_conv2d_fp16_bw_batched(const struct Conv2D_args_fp16 *a, int nsamples);

int ptl_linear_fp32_fw_batched(const struct Linear_args *a, int nsamples);
int ptl_linear_fp32_wg_batched(const struct Linear_args *a, int nsamples);
int ptl_linear_fp32_ig_batched(const struct Linear_args *a, int nsamples);
int ptl_linear_fp16_fw_batched(const struct Linear_args_fp16 *a, int nsamples);
int ptl_linear_fp16_wg_batched(const struct Linear_args_fp16 *a, int nsamples);
int ptl_linear_fp16_ig_batched(const struct Linear_args_fp16 *a, int nsamples);
/* Weight and input gradient of a batch in ONE call, as pulp_linear_fp32_bw_cl /
 * pulp_linear_fp16_bw_cl do for one sample (lib/sources/pulp_linear_fp32.c:67-83,
 * lib/sources/pulp_linear_fp16.c); both products share a launch where they fit. */
int ptl_linear_fp32_bw_batched(const struct Linear_args *a, int nsamples);
int ptl_linear_fp16_bw_batched(const struct Linear_args_fp16 *a, int nsamples);

/* Batched attention step: sample b of every activation blob (input, q, k, v, attention_map,
 * softmax_buffer, output; data and diff) starts b * (rows x columns of that blob) elements in; weights
 * are shared and their gradients are summed over the samples. */
int ptl_mhsa_fp32_fw_batched(const struct Mhsa_args *a, int nsamples);
int ptl_mhsa_fp32_bw_batched(const struct Mhsa_args *a, int nsamples);

/* Batched forms of the layers above: sample b of every activation blob starts b * blob->dim elements
 * in; the loss takes nsamples target vectors and writes nsamples losses.  step: 0 forward, 1 backward;
 * for the residual connection 0 forward, 1 sum node backward, 2 residual backward. */
int ptl_relu_fp32_batched(const struct act_args *a, int nsamples, int step);
int ptl_relu_fp16_batched(const struct act_args_fp16 *a, int nsamples, int step);
int ptl_residual_fp32_batched(const struct SkipConn_args *a, int nsamples, int step);
int ptl_residual_fp16_batched(const struct SkipConn_args_fp16 *a, int nsamples, int step);
int ptl_avgpool_fp32_batched(const struct pool_args *a, int nsamples, int step);
int ptl_avgpool_fp16_batched(const struct pool_args_fp16 *a, int nsamples, int step);
int ptl_cross_entropy_fp32_batched(const struct loss_args *a, int nsamples, int step);
int ptl_cross_entropy_fp16_batched(const struct loss_args_fp16 *a, int nsamples, int step);
int ptl_gradient_descent_fp32(const struct optim_args *a);
int ptl_gradient_descent_fp16(const struct optim_args_fp16 *a);
/* No counterpart in the reference: the update of pulp_gradient_descent_* for `count` argument structs in one
 * launch (a training step updates dozens of small tensors). */
int ptl_gradient_descent_fp32_multi(const struct optim_args *list, int count);
int ptl_gradient_descent_fp16_multi(const struct optim_args_fp16 *list, int count);
/* No counterpart in the reference: forward, weight-gradient and weight + input-gradient calls of a Conv2D batch that
 * share the padded, channel-blocked copy of the layer's input through a caller-owned buffer (struct
 * ptl_conv_cache): the forward call fills it when the layer takes the route that builds such a copy (3x3 fp16
 * channel-major layers with channel counts in multiples of 64; c->valid says whether it did), the gradient calls
 * read it instead of copying the input again.  ptl_conv2d_fp16_cache_bytes returns the size the buffer needs
 * (0: the layer would not use one).  Without a valid cache the calls behave like the plain ones. */
size_t ptl_conv2d_fp16_cache_bytes(const struct Conv2D_args_fp16 *a, int nsamples);
int ptl_conv2d_fp16_fw_batched_cached(const struct Conv2D_args_fp16 *a, int nsamples, struct ptl_conv_cache *c);
int ptl_conv2d_fp16_wg_batched_cached(const struct Conv2D_args_fp16 *a, int nsamples, const struct ptl_conv_cache *c);
int ptl_conv2d_fp16_bw_batched_cached(const struct Conv2D_args_fp16 *a, int nsamples, const struct ptl_conv_cache *c);
/* No counterpart in the reference: layers in a row.  The forward kernel of such a layer can write its output a second
 * time, as the padded, channel-blocked copy the NEXT layer's kernels read, so that the next layer's forward and
 * weight-gradient calls start without their layout pass.  ptl_conv2d_fp16_cache_prepare(reader, ...) sets a cache up
 * as the input copy of the layer `reader` (the caller sets buf - 16-byte aligned device memory - and bytes >=
 * ptl_conv2d_fp16_cache_bytes(reader, nsamples)): it zeroes the buffer once, on the library's stream, and records the
 * geometry; 1 if that layer would not read such a copy.  ptl_conv2d_fp16_fw_batched_chained(a, n, in, out) is the
 * forward call of a layer with `in` = the copy of ITS input (valid: read instead of copying; not valid: filled, as by
 * the _cached call; NULL: none) and `out` = a cache prepared for the layer that reads this layer's output (NULL:
 * none): out->valid says whether the copy was written - the layer must take the resident-tile route and have no
 * bias (USE_BIASES != 1: the bias is added behind the kernel that would write the copy), and its output
 * must be the reader's input tensor (same batch, channels, height and width), or, with out->relu = 1, the input of
 * the ReLU whose output the reader takes: the copy then holds max(output, 0).  The weight-gradient calls of the
 * reader take the same cache through the _cached entry points.  The copies belong to the caller; a call that
 * overlaps another one on the same cache races. */
int ptl_conv2d_fp16_cache_prepare(const struct Conv2D_args_fp16 *reader, int nsamples, struct ptl_conv_cache *c);
int ptl_conv2d_fp16_fw_batched_chained(const struct Conv2D_args_fp16 *a, int nsamples, struct ptl_conv_cache *in,
                                       struct ptl_conv_cache *out);
/* No counterpart in the reference: ptl_conv2d_*_bw_batched with the last launch of a small layer's weight gradient
 * (the addition of its partial sums) put off and done for all deferred layers at once by ptl_conv2d_*_wg_flush
 * (struct ptl_wg_batch; a training step with twenty small layers saves twenty launches).  A layer that does not take
 * the small-layer kernels, finds the batch full, or has its coeff->diff in host memory (a staging copy that the call
 * copies back) is completed by the call itself as usual; with skip_in_grad set the call is the weight-gradient step
 * alone, deferred the same way.  The flush returns 0 also for an empty batch. */
int ptl_conv2d_fp16_bw_batched_deferred(const struct Conv2D_args_fp16 *a, int nsamples, struct ptl_wg_batch *batch);
int ptl_conv2d_fp32_bw_batched_deferred(const struct Conv2D_args *a, int nsamples, struct ptl_wg_batch *batch);
int ptl_conv2d_fp16_wg_flush(struct ptl_wg_batch *batch);
int ptl_conv2d_fp32_wg_flush(struct ptl_wg_batch *batch);
int ptl_batch_norm_fp32_fw(const struct BatchNorm_args_fp32 *a);
/* No counterpart in the reference (its batch normalisation has a forward pass only, in fp32): the backward pass
 * of that forward and both passes in fp16, for a training step that contains the layer.  Backward reads
 * input->data, output->diff, weight_data and eps, writes input->diff (unless skip_in_grad) and, unless
 * skip_wg_grad, the C gradients of the scale into coeff->diff and of the shift into bias->diff (either blob
 * may be NULL). */
int ptl_batch_norm_fp32_bw(const struct BatchNorm_args_fp32 *a);
int ptl_batch_norm_fp16_fw(const struct BatchNorm_args_fp16 *a);
int ptl_batch_norm_fp16_bw(const struct BatchNorm_args_fp16 *a);
/* No counterpart in the reference: the normalisation layer fused with the element-wise layers a residual block
 * puts behind it, for training steps in which those would cost a launch each.
 *   forward:  output->data = [relu]( bn(input->data) [+ f->skip] )
 *   backward: g = output->diff [+ f->diff2], zeroed where output->data <= 0 when f->relu (output->data must still
 *             hold the forward result), rounded to the tensor type; g is written to f->skip_diff when that is
 *             given (the gradient of the skip branch); input->diff, coeff->diff and bias->diff as
 *             ptl_batch_norm_*_bw computes them from g. */
int ptl_batch_norm_fused_fp32_fw(const struct BatchNorm_args_fp32 *a, const struct ptl_norm_fusion_fp32 *f);
int ptl_batch_norm_fused_fp32_bw(const struct BatchNorm_args_fp32 *a, const struct ptl_norm_fusion_fp32 *f);
int ptl_batch_norm_fused_fp16_fw(const struct BatchNorm_args_fp16 *a, const struct ptl_norm_fusion_fp16 *f);
int ptl_batch_norm_fused_fp16_bw(const struct BatchNorm_args_fp16 *a, const struct ptl_norm_fusion_fp16 *f);
/* No counterpart in the reference: the forward convolution that also leaves the sums a batch normalisation of its
 * output needs (struct ptl_norm_stats; formed from the values as stored, inside the small-layer kernels - other
 * layers, and layers with USE_BIASES, return with st->valid = 0), and the fused normalisation forward that takes
 * them: with st->valid and matching channels and count it runs one launch instead of two, else it behaves like
 * ptl_batch_norm_fused_*_fw (f may be NULL: no fusion).  The sums are added in another order than the
 * normalisation's own, so results agree to rounding of the statistics, not bit for bit. */
int ptl_conv2d_fp32_fw_batched_stats(const struct Conv2D_args *a, int nsamples, struct ptl_norm_stats *st);
int ptl_conv2d_fp16_fw_batched_stats(const struct Conv2D_args_fp16 *a, int nsamples, struct ptl_norm_stats *st);
int ptl_batch_norm_fused_fp32_fw_stats(const struct BatchNorm_args_fp32 *a, const struct ptl_norm_fusion_fp32 *f,
                                       const struct ptl_norm_stats *st);
int ptl_batch_norm_fused_fp16_fw_stats(const struct BatchNorm_args_fp16 *a, const struct ptl_norm_fusion_fp16 *f,
                                       const struct ptl_norm_stats *st);
/* No counterpart in the reference: the tail of a classifier and its way back in one call - ptl_avgpool_*_batched(pool,
 * n, 0), ptl_linear_*_fw_batched(lin, n), ptl_cross_entropy_*_batched(loss, n, 0) and (loss, n, 1),
 * ptl_linear_*_bw_batched(lin, n), ptl_avgpool_*_batched(pool, n, 1), every tensor those calls write included.  One
 * launch when the pooling is global (window = plane), its output blob is the classifier's input and the
 * classifier's output blob the loss's (same data and diff pointers), at most 32 classes, no bias, both gradients
 * wanted, device tensors, and `batch` (a struct ptl_wg_batch, see ptl_conv2d_*_bw_batched_deferred) has room: the
 * classifier's weight gradient is then complete after the flush, like a deferred convolution's.  Results agree with
 * the six calls to rounding (the dot products are added up in another order).  Anything else: the six calls. */
int ptl_pool_linear_loss_fp32_batched(const struct pool_args *pool, const struct Linear_args *lin, const struct loss_args *loss,
                                      int nsamples, struct ptl_wg_batch *batch);
int ptl_pool_linear_loss_fp16_batched(const struct pool_args_fp16 *pool, const struct Linear_args_fp16 *lin,
                                      const struct loss_args_fp16 *loss, int nsamples, struct ptl_wg_batch *batch);
/* No counterpart in the reference: ptl_batch_norm_fused_*_fw_stats(norm, f, norm_st) followed by
 * ptl_conv2d_*_fw_batched_stats(a, nsamples, st) (st may be NULL: no sums wanted) for a convolution that reads the
 * normalisation's output (norm->output->data == a->input->data) - same results bit for bit, the normalisation's
 * output tensor included.  Where the small-layer kernel takes the convolution (device tensors, valid norm_st, every
 * input row read by the tile that starts at it: unit or double stride with "same" padding) it is one launch: the
 * kernel normalises its input tile while it loads it and writes the normalisation's output on the way. */
int ptl_conv2d_fp32_fw_batched_normed(const struct Conv2D_args *a, int nsamples, struct ptl_norm_stats *st,
                                      const struct BatchNorm_args_fp32 *norm, const struct ptl_norm_fusion_fp32 *f,
                                      const struct ptl_norm_stats *norm_st);
int ptl_conv2d_fp16_fw_batched_normed(const struct Conv2D_args_fp16 *a, int nsamples, struct ptl_norm_stats *st,
                                      const struct BatchNorm_args_fp16 *norm, const struct ptl_norm_fusion_fp16 *f,
                                      const struct ptl_norm_stats *norm_st);
/* No counterpart in the reference: the backward twin of the pair above.  The one-call backward of the convolution
 * BEHIND a normalisation forms, in the epilogue of its input gradient, the gradient g that the normalisation's
 * backward pass starts from (struct ptl_grad_post: g = (dX [+ add]) [where mask > 0, else 0]) and the sums of g and
 * g * x per channel; sums->valid says whether it did (the small-layer kernel on device tensors: unit stride, at most
 * 64 channels and filters; otherwise input->diff is the plain input gradient and valid is 0).  Host tensors are
 * rejected (status 1).
 * ptl_batch_norm_fused_*_bw_stats is the normalisation's backward call behind it.  With bw->valid == 1 it takes
 * output->diff as g - nothing added, nothing masked, f ignored - and, when fw (the forward sums of the
 * normalisation's input, still in their buffer) is valid too, runs one launch instead of two.  With bw NULL or not
 * valid it is ptl_batch_norm_fused_*_bw with f: describe the same addition and mask there (f->diff2 = post->add,
 * f->relu with output->data = post->mask) and let f->skip_diff be output->diff, so that g ends up in output->diff
 * either way. */
int ptl_conv2d_fp32_bw_batched_deferred_post(const struct Conv2D_args *a, int nsamples, struct ptl_wg_batch *batch,
                                             const struct ptl_grad_post *post, struct ptl_norm_stats *sums);
int ptl_conv2d_fp16_bw_batched_deferred_post(const struct Conv2D_args_fp16 *a, int nsamples, struct ptl_wg_batch *batch,
                                             const struct ptl_grad_post *post, struct ptl_norm_stats *sums);
int ptl_batch_norm_fused_fp32_bw_stats(const struct BatchNorm_args_fp32 *a, const struct ptl_norm_fusion_fp32 *f,
                                       const struct ptl_norm_stats *fw, const struct ptl_norm_stats *bw);
int ptl_batch_norm_fused_fp16_bw_stats(const struct BatchNorm_args_fp16 *a, const struct ptl_norm_fusion_fp16 *f,
                                       const struct ptl_norm_stats *fw, const struct ptl_norm_stats *bw);

/* Plain product C[N x M] = A[N x K] * B (B is K x M, or M x K when trans_B),
 * the contract of the reference's mm family, on raw pointers. */
int ptl_mm_fp32(const float *A, const float *B, float *C, int N, int M, int K, int trans_B);
int ptl_mm_fp16(const fp16 *A, const fp16 *B, fp16 *C, int N, int M, int K, int trans_B);

/* Device-to-device copy kernel of `bytes` bytes (multiple of 16), used to
 * calibrate memory-traffic counters against a known size. */
int ptl_copy_bytes(const void *src, void *dst, long bytes);

#ifdef __cplusplus
}
#endif
#endif /* PTL_API_H */
