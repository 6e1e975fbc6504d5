/*
 * Argument structures of the matmul-based training core, laid out field for
 * field like the PULP-TrainLib structures they stand in for, so that a caller
 * compiled against the PULP-TrainLib headers can hand its structs to this
 * library unchanged.  Every struct names the reference declaration it mirrors.
 *
 * Only the data layout is shared with the reference; the code behind the
 * entry points is HIP for gfx950.
 */
#ifndef PTL_STRUCTS_H
#define PTL_STRUCTS_H

#include <stdint.h>

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/* IEEE binary16 storage type.  The reference picks its 16-bit format with a
 * typedef (lib/include/pulp_train_defines.h:32: float16alt by default, float16
 * as the documented alternative); this library implements the IEEE `float16`
 * option, which is what the gfx950 fp16 MFMA consumes.  Host code in this
 * library never does arithmetic on fp16 values, so a compiler without _Float16
 * may use a same-sized integer. */
#if defined(__FLT16_MANT_DIG__)
typedef _Float16 fp16;
#else
typedef uint16_t fp16;
#endif

/* Step and layer selectors of mm_manager (lib/include/pulp_train_defines.h:51-65). */
#define LAYER_CONV2D 0
#define LAYER_DW_CONV 1
#define LAYER_PW_CONV 2
#define LAYER_LINEAR 3
#define STEP_FW 0
#define STEP_WGT_GRAD 1
#define STEP_IN_GRAD 2

/* Tensor + gradient handle (lib/include/pulp_train_utils_fp32.h:37-44).
 * For a weight blob W,H are the kernel size and C the input channels. */
struct blob {
    float *data;
    float *diff;
    int dim;
    int W;
    int H;
    int C;
};

/* lib/include/pulp_train_utils_fp16.h:38-45 */
struct blob_fp16 {
    fp16 *data;
    fp16 *diff;
    int dim;
    int W;
    int H;
    int C;
};

/* lib/include/pulp_train_utils_fp32.h:63-77 */
struct im2col_args {
    struct blob *input;
    struct blob *c;
    struct blob *output;
    float *pBuffer;
    int Lpad;
    int Rpad;
    int Upad;
    int Dpad;
    int mod;
    int stride_w;
    int stride_h;
    int HWC;
    int USE_DMA;
};

/* lib/include/pulp_train_utils_fp16.h:64-78 */
struct im2col_args_fp16 {
    struct blob_fp16 *input;
    struct blob_fp16 *c;
    struct blob_fp16 *output;
    fp16 *pBuffer;
    int Lpad;
    int Rpad;
    int Upad;
    int Dpad;
    int mod;
    int stride_w;
    int stride_h;
    int HWC;
    int USE_DMA;
};

/* lib/include/pulp_train_utils_fp32.h:91-99 */
struct transp_args {
    float *in_matrix;
    float *out_matrix;
    int N;
    int M;
    int *dim;
    int *transposed_axes;
    int n_dim;
};

/* lib/include/pulp_train_utils_fp16.h:93-101 */
struct transp_args_fp16 {
    fp16 *in_matrix;
    fp16 *out_matrix;
    int N;
    int M;
    int *dim;
    int *transposed_axes;
    int n_dim;
};

/* lib/include/pulp_train_utils_fp32.h:109-114 */
struct layout_args {
    struct blob *tensor;
    float *transp_buffer;
    int transpose_data;
    int transpose_grad;
};

/* lib/include/pulp_train_utils_fp16.h:133-138 */
struct layout_args_fp16 {
    struct blob_fp16 *tensor;
    fp16 *transp_buffer;
    int transpose_data;
    int transpose_grad;
};

/* lib/include/pulp_train_utils_fp32.h:127-135 */
struct blocktransp_args {
    float *weights;
    float *bt_weights;
    int Cin;
    int Cout;
    int Hk;
    int Wk;
    int HWC;
};

/* lib/include/pulp_train_utils_fp16.h:150-158 */
struct blocktransp_args_fp16 {
    fp16 *weights;
    fp16 *bt_weights;
    int Cin;
    int Cout;
    int Hk;
    int Wk;
    int HWC;
};

/* lib/include/pulp_train_utils_fp32.h:144-148 */
struct copy_args {
    float *from;
    float *to;
    int size;
};

/* lib/include/pulp_train_utils_fp16.h:167-171 */
struct copy_args_fp16 {
    fp16 *from;
    fp16 *to;
    int size;
};

/* lib/include/pulp_train_utils_fp32.h:157-161 */
struct set_to_value_args {
    float *to;
    float value;
    int size;
};

/* lib/include/pulp_train_utils_fp16.h:180-184 */
struct set_to_value_args_fp16 {
    fp16 *to;
    fp16 value;
    int size;
};

/* lib/include/pulp_train_utils_fp32.h:171-176 */
struct vect_sum_args {
    float *op_1;
    float *op_2;
    float *dest;
    int size;
};

/* lib/include/pulp_train_utils_fp16.h:194-199 */
struct vect_sum_args_fp16 {
    fp16 *op_1;
    fp16 *op_2;
    fp16 *dest;
    int size;
};

/* lib/include/pulp_train_utils_fp32.h:206-210 */
struct cast_16t32_args {
    fp16 *source;
    float *destination;
    int size;
};

/* lib/include/pulp_train_utils_fp16.h:208-212 */
struct cast_32t16_args {
    float *source;
    fp16 *destination;
    int size;
};

/* lib/include/pulp_train_utils_fp32.h:226-237 (note: RPAD precedes LPAD) */
struct pad_args {
    float *source;
    float *dest;
    int C;
    int H;
    int W;
    int T_RPAD;
    int T_LPAD;
    int T_UPAD;
    int T_DPAD;
    int HWC_lay;
};

/* lib/include/pulp_train_utils_fp16.h:228-239 */
struct pad_args_fp16 {
    fp16 *source;
    fp16 *dest;
    int C;
    int H;
    int W;
    int T_RPAD;
    int T_LPAD;
    int T_UPAD;
    int T_DPAD;
    int HWC_lay;
};

/* GEMM descriptor C[N x M] = A[N x K] * B, with B stored K x M (trans_B = 0)
 * or M x K (trans_B = 1)  (lib/include/pulp_train_utils_fp32.h:268-297). */
struct matMul_args {
    float *A;
    float *B;
    float *C;
    int N;
    int M;
    int K;
    int trans_B;

    int H;
    int W;
    int pW;
    int pH;
    int pCin;
    int pCout;
    int stride_h;
    int stride_w;
    int Lpad;
    int Rpad;
    int Upad;
    int Dpad;

    float *bias;
    int bias_dim;
    int USE_BIASES;
    int bias_transposed;
    int HWC;
};

/* lib/include/pulp_train_utils_fp16.h:292-321 */
struct matMul_args_fp16 {
    fp16 *A;
    fp16 *B;
    fp16 *C;
    int N;
    int M;
    int K;
    int trans_B;

    int H;
    int W;
    int pW;
    int pH;
    int pCin;
    int pCout;
    int stride_h;
    int stride_w;
    int Lpad;
    int Rpad;
    int Upad;
    int Dpad;

    fp16 *bias;
    int bias_dim;
    int USE_BIASES;
    int bias_transposed;
    int HWC;
};

/* lib/include/pulp_train_utils_fp32.h:338-351 */
struct kernel_DW_args {
    struct blob *input;
    struct blob *weights;
    struct blob *output;
    int stride_h;
    int stride_w;
    int Lpad;
    int Rpad;
    int Upad;
    int Dpad;
};

/* lib/include/pulp_train_utils_fp16.h:330-334 */
struct kernel_DW_args_fp16 {
    struct blob_fp16 *input;
    struct blob_fp16 *weights;
    struct blob_fp16 *output;
};

struct matMul_DW_args;      /* never dereferenced on this path */
struct matMul_DW_args_fp16; /* never dereferenced on this path */

/* lib/include/pulp_train_utils_fp32.h:360-366 */
struct mm_manager_args {
    struct matMul_args *mm_args;
    struct matMul_DW_args *mm_dw_args;
    int layer_type;
    int step_type;
    int matmul_type;
};

/* lib/include/pulp_train_utils_fp16.h:345-351 */
struct mm_manager_args_fp16 {
    struct matMul_args_fp16 *mm_args;
    struct matMul_DW_args_fp16 *mm_dw_args;
    int layer_type;
    int step_type;
    int matmul_type;
};

/* lib/include/pulp_train_utils_fp32.h:569-575 */
struct mm_bias_add_args {
    float *mat;
    float *bias;
    int H;
    int W;
    int t;
};

/* lib/include/pulp_train_utils_fp16.h:524-530 */
struct mm_bias_add_args_fp16 {
    fp16 *mat;
    fp16 *bias;
    int H;
    int W;
    int t;
};

/* lib/include/pulp_conv2d_fp32.h:50-72 */
struct Conv2D_args {
    struct blob *input;
    struct blob *coeff;
    struct blob *bias;
    struct blob *output;
    int Lpad;
    int Rpad;
    int Upad;
    int Dpad;
    int stride_h;
    int stride_w;
    float *i2c_buffer;
    float *bt_buffer;
    int skip_wg_grad;
    int skip_in_grad;
    int HWC;
    int opt_matmul_type_fw;
    int opt_matmul_type_wg;
    int opt_matmul_type_ig;
    int USE_BIASES;
    int USE_IM2COL;
    int USE_DMA_IM2COL;
};

/* lib/include/pulp_conv2d_fp16.h:51-73 */
struct Conv2D_args_fp16 {
    struct blob_fp16 *input;
    struct blob_fp16 *coeff;
    struct blob_fp16 *bias;
    struct blob_fp16 *output;
    int Lpad;
    int Rpad;
    int Upad;
    int Dpad;
    int stride_h;
    int stride_w;
    fp16 *i2c_buffer;
    fp16 *bt_buffer;
    int skip_wg_grad;
    int skip_in_grad;
    int HWC;
    int opt_matmul_type_fw;
    int opt_matmul_type_wg;
    int opt_matmul_type_ig;
    int USE_BIASES;
    int USE_IM2COL;
    int USE_DMA_IM2COL;
};

/* lib/include/pulp_conv_pw_fp32.h:39-50 */
struct PointWise_Conv_args {
    struct blob *input;
    struct blob *coeff;
    struct blob *output;
    float *transpose_buffer;
    int skip_wg_grad;
    int skip_in_grad;
    int opt_matmul_type_fw;
    int opt_matmul_type_wg;
    int opt_matmul_type_ig;
    int HWC;
};

/* lib/include/pulp_conv_pw_fp16.h:40-51 */
struct PointWise_Conv_args_fp16 {
    struct blob_fp16 *input;
    struct blob_fp16 *coeff;
    struct blob_fp16 *output;
    fp16 *transpose_buffer;
    int skip_wg_grad;
    int skip_in_grad;
    int opt_matmul_type_fw;
    int opt_matmul_type_wg;
    int opt_matmul_type_ig;
    int HWC;
};

/* lib/include/pulp_conv_dw_fp32.h:43-60 */
struct DepthWise_Conv_args {
    struct blob *input;
    struct blob *coeff;
    struct blob *output;
    int stride_h;
    int stride_w;
    int Lpad;
    int Rpad;
    int Upad;
    int Dpad;
    int skip_wg_grad;
    int skip_in_grad;
    int HWC;
};

/* lib/include/pulp_conv_dw_fp16.h:40-51 (no stride fields) */
struct DepthWise_Conv_args_fp16 {
    struct blob_fp16 *input;
    struct blob_fp16 *coeff;
    struct blob_fp16 *output;
    int Lpad;
    int Rpad;
    int Upad;
    int Dpad;
    int skip_wg_grad;
    int skip_in_grad;
    int HWC;
};

/* lib/include/pulp_linear_fp32.h:39-50 */
struct Linear_args {
    struct blob *input;
    struct blob *coeff;
    struct blob *bias;
    struct blob *output;
    int skip_wg_grad;
    int skip_in_grad;
    int opt_matmul_type_fw;
    int opt_matmul_type_wg;
    int opt_matmul_type_ig;
    int use_biases;
};

/* lib/include/pulp_linear_fp16.h:39-50 */
struct Linear_args_fp16 {
    struct blob_fp16 *input;
    struct blob_fp16 *coeff;
    struct blob_fp16 *bias;
    struct blob_fp16 *output;
    int skip_wg_grad;
    int skip_in_grad;
    int opt_matmul_type_fw;
    int opt_matmul_type_wg;
    int opt_matmul_type_ig;
    int use_biases;
};

/* Row-wise softmax (lib/include/pulp_act_fp32.h:53-66).  H rows of W elements;
 * `maxes` and `sums` are H-element scratch rows the forward pass fills. */
struct softmax_args {
    float *input_data;
    float *input_diff;
    float *output_data;
    float *output_diff;
    int H;
    int W;
    int L;
    int n_heads;
    float *global_max;
    float *partial_exp_sum;
    float *maxes;
    float *sums;
};

/* Multi-head self-attention (lib/include/pulp_mhsa_fp32.h:52-83).
 * With L = input->H (sequence length), E = input->W (token size),
 * F = attention_map->W (heads x head size):
 *   input, output            E x L   (tokens are columns)
 *   coeff_in_q/k/v  data     E x F   (transposed projection weights), diff F x E
 *   bias_in_q/k/v   data     F
 *   coeff_out                E x F   (data and diff)
 *   q, k, v, attention_map   F x L   (data and diff)
 *   softmax_buffer           n_heads x L x L, row = query, column = key (data and diff)
 * temp_buffer, grad, sums, maxes, head_buffer, input_bn, bias_out, global_max and
 * partial_exp_sum are scratch or unused on this path. */
struct Mhsa_args {
    struct blob *input;
    struct blob *input_bn;
    int n_heads;
    int opt_matmul_type_fw;
    int opt_matmul_type_wg;
    int opt_matmul_type_ig;
    struct blob *output;
    struct blob *coeff_in_q;
    struct blob *coeff_in_k;
    struct blob *coeff_in_v;
    struct blob *bias_in_q;
    struct blob *bias_in_k;
    struct blob *bias_in_v;
    struct blob *coeff_out;
    struct blob *bias_out;
    struct blob *q;
    struct blob *k;
    struct blob *v;
    struct blob *attention_map;
    float *temp_buffer;
    float *grad;
    struct blob *head_buffer;
    struct blob *softmax_buffer;
    float *global_max;
    float *partial_exp_sum;
    float *maxes;
    float *sums;
};

/* ---- Layers around the matmul core in a ResNet-style training step ---- */

/* Activation (lib/include/pulp_act_fp32.h:27-32, pulp_act_fp16.h:28-33): input->dim elements. */
struct act_args {
    struct blob *input;
    struct blob *output;
    int H;
    int W;
};
struct act_args_fp16 {
    struct blob_fp16 *input;
    struct blob_fp16 *output;
    int H;
    int W;
};

/* Residual connection (lib/include/pulp_residual_fp32.h:50-55, pulp_residual_fp16.h:50-55). */
struct SkipConn_args {
    struct blob *skip;
    struct blob *lout;
    struct blob *output;
    int skip_in_grad;
};
struct SkipConn_args_fp16 {
    struct blob_fp16 *skip;
    struct blob_fp16 *lout;
    struct blob_fp16 *output;
    int skip_in_grad;
};

/* Pooling (lib/include/pulp_pooling_fp32.h:34-41, pulp_pooling_fp16.h:34-41). */
struct pool_args {
    struct blob *input;
    struct blob *output;
    int Hker;
    int Wker;
    int Hstride;
    int Wstride;
};
struct pool_args_fp16 {
    struct blob_fp16 *input;
    struct blob_fp16 *output;
    int Hker;
    int Wker;
    int Hstride;
    int Wstride;
};

/* Loss (lib/include/pulp_losses_fp32.h:32-36, pulp_losses_fp16.h:33-37): output->data are the logits,
 * output->diff receives their gradient, target is a one-hot (or soft) vector of output->dim classes. */
struct loss_args {
    struct blob *output;
    float *target;
    float *wr_loss;
};
struct loss_args_fp16 {
    struct blob_fp16 *output;
    fp16 *target;
    fp16 *wr_loss;
};

/* Gradient descent (lib/include/pulp_optimizers_fp32.h:34-40, pulp_optimizers_fp16.h:35-41). */
struct optim_args {
    struct blob *weights;
    struct blob *biases;
    float learning_rate;
    float weight_decay_lambda;
    int use_biases;
};
struct optim_args_fp16 {
    struct blob_fp16 *weights;
    struct blob_fp16 *biases;
    fp16 learning_rate;
    fp16 weight_decay_lambda;
    int use_biases;
};

/* Batch normalisation, forward only (lib/include/pulp_batchnorm_fp32.h:40-66): statistics per channel
 * over B x H x W; the forward pass reads input, output, weight_data, bias_data, eps and B, C, H, W. */
struct BatchNorm_args_fp32 {
    struct blob *input;
    struct blob *output;
    struct blob *coeff;
    struct blob *bias;
    int batch_size;
    float *running_mean;
    float *running_var;
    float *running_stdev;
    int freeze_running_params;
    int skip_wg_grad;
    int skip_in_grad;
    float *weight_data;
    float *bias_data;
    float *eps;
    int B;
    int C;
    int H;
    int W;
};

/* The same in fp16 (no counterpart in the reference, which normalises in fp32 only): tensors, affine
 * parameters and eps in fp16, statistics in fp32. */
struct BatchNorm_args_fp16 {
    struct blob_fp16 *input;
    struct blob_fp16 *output;
    struct blob_fp16 *coeff;
    struct blob_fp16 *bias;
    int batch_size;
    float *running_mean;
    float *running_var;
    float *running_stdev;
    int freeze_running_params;
    int skip_wg_grad;
    int skip_in_grad;
    fp16 *weight_data;
    fp16 *bias_data;
    fp16 *eps;
    int B;
    int C;
    int H;
    int W;
};

/* No counterpart in the reference: a caller-owned buffer in which a Conv2D forward call leaves its padded,
 * channel-blocked copy of the layer's input for the weight-gradient call of the same layer on the same input
 * (ptl_conv2d_fp16_*_cached).  The caller sets buf and bytes (ptl_conv2d_fp16_cache_bytes) and keeps both alive and
 * the input unchanged between the two calls; the library writes valid and geometry. */
struct ptl_conv_cache {
    void *buf;
    size_t bytes;
    int valid;       /* 1: buf holds the copy described by geometry */
    int geometry[6]; /* batch, channels, padded height and width, top and left padding */
    int relu;        /* set by the caller, read by ptl_conv2d_fp16_fw_batched_chained when it writes this cache as the
                        copy of its OUTPUT: 1 = write max(output, 0), for a reader that sits behind a ReLU */
};

/* No counterpart in the reference: the weight gradients of several small Conv2D layers completed by one launch.
 * A backward call of such a layer is two launches, the second one only adds up the partial sums of the first;
 * with a batch (ptl_conv2d_*_bw_batched_deferred) the partial sums stay in the caller's buffer and
 * ptl_conv2d_*_wg_flush adds up those of all layers deferred since the last flush.  The caller sets buf and bytes
 * (device memory, 16 MiB hold the layers of a ResNet-20 at batch 128) and zeroes used and count once; the library
 * maintains the rest.  coeff->diff of a deferred layer is valid after the flush, not before. */
#define PTL_WG_BATCH_MAX 32
struct ptl_wg_batch {
    void *buf;
    size_t bytes;
    size_t used;      /* bytes of buf in use */
    int count;        /* layers waiting for the flush */
    size_t offset[32]; /* per layer: where its partial sums start in buf */
    void *grad[32];    /* per layer: its coeff->diff */
    int shape[256];    /* per layer eight numbers: floats per part, parts, filter rows and channels kept of a 32 x 32
                          tile, channel blocks, filters, channels, taps */
};

/* No counterpart in the reference: sums of a convolution's output and of its squares per channel, left by
 * ptl_conv2d_*_fw_batched_stats for the batch normalisation behind it (ptl_batch_norm_fused_*_fw_stats), which then
 * skips the launch that would read the tensor again for them.  The caller provides part (device memory, 16-byte
 * aligned; 16 bytes per channel and workgroup of the convolution, 1 MiB hold any layer of a ResNet-20 at batch 128);
 * the convolution fills the rest and sets valid to 1 when it took a route that forms the sums, else to 0. */
struct ptl_norm_stats {
    float *part;    /* [channel][part][4]: sum, sum of squares, two unused */
    size_t bytes;   /* size of part */
    size_t count;   /* elements per channel the sums cover (samples x rows x columns) */
    int parts;      /* partial sums per channel */
    int channels;
    int valid;
};

/* No counterpart in the reference: what a residual block puts behind a normalisation layer, for the fused calls
 * ptl_batch_norm_fused_*.  All tensors have the shape of the normalisation's output (B x C x H x W). */
struct ptl_norm_fusion_fp32 {
    int relu;          /* 1: ReLU after the (optional) addition */
    const float *skip; /* forward: tensor added to the normalised input; NULL: none */
    float *skip_diff;  /* backward: receives the gradient of the sum (= of the skip tensor); NULL: not wanted */
    const float *diff2; /* backward: a second incoming gradient, added to output->diff; NULL: none */
};
struct ptl_norm_fusion_fp16 {
    int relu;
    const fp16 *skip;
    fp16 *skip_diff;
    const fp16 *diff2;
};

/* No counterpart in the reference: what stands between a convolution's input gradient and the backward pass of the
 * batch normalisation in front of that convolution, done in the convolution's epilogue
 * (ptl_conv2d_*_bw_batched_deferred_post).  All tensors have the shape of the convolution's input (device memory):
 *   g = input->diff as the call computes it [+ add], rounded to the tensor type, [zeroed where mask <= 0];
 * g is what the call stores to input->diff, and the sums of g and of g * x per channel go to a struct
 * ptl_norm_stats (part[..][0] and [1]).  x is the normalisation's input (its sums need it), mask its output when a
 * ReLU follows it, add a second incoming gradient (the shortcut's). */
struct ptl_grad_post {
    const void *add;  /* NULL: none */
    const void *mask; /* NULL: no ReLU */
    const void *x;
};

#ifdef __cplusplus
}
#endif
#endif /* PTL_STRUCTS_H */
