/*
 * The reference's entry points, in C, over the HIP launchers.
 *
 * Every function here has the name, the `void f(void *args)` signature and
 * the argument struct of the PULP-TrainLib function it replaces; the body
 * translates the struct into one or two calls of the batched launchers with
 * a single sample.  Where the reference forks a kernel on NUM_CORES cluster
 * cores, the launcher enqueues one grid on the GPU.
 *
 * The reference reports nothing to its caller: a rejected call prints a
 * message and leaves the outputs untouched.  That is kept; in addition the
 * outcome of the last call is readable through ptl_last_status().
 */
#include <stddef.h>
#include <stdio.h>

#include "ptl_api.h"
#include "ptl_internal.h"

/* ---- Conv2D (lib/sources/pulp_conv2d_fp32.c, pulp_conv2d_fp16.c) ---------- */

void pulp_conv2d_fp32_fw_cl(void *p) { ptl_internal_set_status(ptl_conv2d_fp32_fw_batched(p, 1)); }
void pulp_conv2d_fp32_bw_param_grads_cl(void *p) { ptl_internal_set_status(ptl_conv2d_fp32_wg_batched(p, 1)); }
void pulp_conv2d_fp32_bw_input_grads_cl(void *p) { ptl_internal_set_status(ptl_conv2d_fp32_ig_batched(p, 1)); }

/* Both gradients unless skipped (lib/sources/pulp_conv2d_fp32.c:225-237). */
void pulp_conv2d_fp32_bw_cl(void *p) {
    struct Conv2D_args *a = (struct Conv2D_args *)p;
    int rc = 0;
    if (a && a->skip_wg_grad == 0) rc = ptl_conv2d_fp32_wg_batched(a, 1);
    if (a && a->skip_in_grad == 0) {
        int r2 = ptl_conv2d_fp32_ig_batched(a, 1);
        if (rc == 0) rc = r2;
    }
    ptl_internal_set_status(a ? rc : 1);
}

void pulp_conv2d_fp16_fw_cl(void *p) { ptl_internal_set_status(ptl_conv2d_fp16_fw_batched(p, 1)); }
void pulp_conv2d_fp16_bw_param_grads_cl(void *p) { ptl_internal_set_status(ptl_conv2d_fp16_wg_batched(p, 1)); }
void pulp_conv2d_fp16_bw_input_grads_cl(void *p) { ptl_internal_set_status(ptl_conv2d_fp16_ig_batched(p, 1)); }

void pulp_conv2d_fp16_bw_cl(void *p) {
    struct Conv2D_args_fp16 *a = (struct Conv2D_args_fp16 *)p;
    int rc = 0;
    if (a && a->skip_wg_grad == 0) rc = ptl_conv2d_fp16_wg_batched(a, 1);
    if (a && a->skip_in_grad == 0) {
        int r2 = ptl_conv2d_fp16_ig_batched(a, 1);
        if (rc == 0) rc = r2;
    }
    ptl_internal_set_status(a ? rc : 1);
}

/* ---- Pointwise (lib/sources/pulp_conv_pw_fp32.c, pulp_conv_pw_fp16.c) ------ */

void pulp_conv_pw_fp32_fw_cl(void *p) { ptl_internal_set_status(ptl_conv_pw_fp32_fw_batched(p, 1)); }
void pulp_conv_pw_fp32_bw_param_grads_cl(void *p) { ptl_internal_set_status(ptl_conv_pw_fp32_wg_batched(p, 1)); }
void pulp_conv_pw_fp32_bw_input_grads_cl(void *p) { ptl_internal_set_status(ptl_conv_pw_fp32_ig_batched(p, 1)); }

void pulp_conv_pw_fp32_bw_cl(void *p) {
    struct PointWise_Conv_args *a = (struct PointWise_Conv_args *)p;
    int rc = 0;
    if (a && a->skip_wg_grad == 0) rc = ptl_conv_pw_fp32_wg_batched(a, 1);
    if (a && a->skip_in_grad == 0) {
        int r2 = ptl_conv_pw_fp32_ig_batched(a, 1);
        if (rc == 0) rc = r2;
    }
    ptl_internal_set_status(a ? rc : 1);
}

void pulp_conv_pw_fp16_fw_cl(void *p) { ptl_internal_set_status(ptl_conv_pw_fp16_fw_batched(p, 1)); }
void pulp_conv_pw_fp16_bw_param_grads_cl(void *p) { ptl_internal_set_status(ptl_conv_pw_fp16_wg_batched(p, 1)); }
void pulp_conv_pw_fp16_bw_input_grads_cl(void *p) { ptl_internal_set_status(ptl_conv_pw_fp16_ig_batched(p, 1)); }

void pulp_conv_pw_fp16_bw_cl(void *p) {
    struct PointWise_Conv_args_fp16 *a = (struct PointWise_Conv_args_fp16 *)p;
    int rc = 0;
    if (a && a->skip_wg_grad == 0) rc = ptl_conv_pw_fp16_wg_batched(a, 1);
    if (a && a->skip_in_grad == 0) {
        int r2 = ptl_conv_pw_fp16_ig_batched(a, 1);
        if (rc == 0) rc = r2;
    }
    ptl_internal_set_status(a ? rc : 1);
}

/* ---- Depthwise (lib/sources/pulp_conv_dw_fp32.c, pulp_conv_dw_fp16.c) ------ */

void pulp_conv_dw_fp32_fw_cl(void *p) { ptl_internal_set_status(ptl_conv_dw_fp32_fw_batched(p, 1)); }
void pulp_conv_dw_fp32_bw_param_grads_cl(void *p) { ptl_internal_set_status(ptl_conv_dw_fp32_wg_batched(p, 1)); }
void pulp_conv_dw_fp32_bw_input_grads_cl(void *p) { ptl_internal_set_status(ptl_conv_dw_fp32_ig_batched(p, 1)); }

void pulp_conv_dw_fp32_bw_cl(void *p) {
    struct DepthWise_Conv_args *a = (struct DepthWise_Conv_args *)p;
    int rc = 0;
    if (a && a->skip_wg_grad == 0) rc = ptl_conv_dw_fp32_wg_batched(a, 1);
    if (a && a->skip_in_grad == 0) {
        int r2 = ptl_conv_dw_fp32_ig_batched(a, 1);
        if (rc == 0) rc = r2;
    }
    ptl_internal_set_status(a ? rc : 1);
}

void pulp_conv_dw_fp16_fw_cl(void *p) { ptl_internal_set_status(ptl_conv_dw_fp16_fw_batched(p, 1)); }
void pulp_conv_dw_fp16_bw_param_grads_cl(void *p) { ptl_internal_set_status(ptl_conv_dw_fp16_wg_batched(p, 1)); }
void pulp_conv_dw_fp16_bw_input_grads_cl(void *p) { ptl_internal_set_status(ptl_conv_dw_fp16_ig_batched(p, 1)); }

void pulp_conv_dw_fp16_bw_cl(void *p) {
    struct DepthWise_Conv_args_fp16 *a = (struct DepthWise_Conv_args_fp16 *)p;
    int rc = 0;
    if (a && a->skip_wg_grad == 0) rc = ptl_conv_dw_fp16_wg_batched(a, 1);
    if (a && a->skip_in_grad == 0) {
        int r2 = ptl_conv_dw_fp16_ig_batched(a, 1);
        if (rc == 0) rc = r2;
    }
    ptl_internal_set_status(a ? rc : 1);
}

/* The kernels the depthwise layer forks (lib/sources/pulp_conv_naive_fp32.c:29,
 * :113, :153).  The fp16 kernel struct carries no padding or stride
 * (lib/include/pulp_train_utils_fp16.h:330-334). */
static void dw_from_kernel_args(const struct kernel_DW_args *k, struct DepthWise_Conv_args *a) {
    a->input = k->input;
    a->coeff = k->weights;
    a->output = k->output;
    a->stride_h = k->stride_h;
    a->stride_w = k->stride_w;
    a->Lpad = k->Lpad;
    a->Rpad = k->Rpad;
    a->Upad = k->Upad;
    a->Dpad = k->Dpad;
    a->skip_wg_grad = 0;
    a->skip_in_grad = 0;
    a->HWC = 0;
}

void dw_kernel_forward(void *p) {
    struct DepthWise_Conv_args a;
    if (!p) { ptl_internal_set_status(1); return; }
    dw_from_kernel_args((const struct kernel_DW_args *)p, &a);
    ptl_internal_set_status(ptl_conv_dw_fp32_fw_batched(&a, 1));
}

/* The reference's weight- and input-gradient kernels read neither stride nor
 * padding (unit stride, no padding); the struct fields are passed on so that a
 * caller who does set them gets the gradient of the forward it ran. */
void dw_kernel_weight_grad(void *p) {
    struct DepthWise_Conv_args a;
    if (!p) { ptl_internal_set_status(1); return; }
    dw_from_kernel_args((const struct kernel_DW_args *)p, &a);
    ptl_internal_set_status(ptl_conv_dw_fp32_wg_batched(&a, 1));
}

void dw_kernel_input_grad(void *p) {
    struct DepthWise_Conv_args a;
    if (!p) { ptl_internal_set_status(1); return; }
    dw_from_kernel_args((const struct kernel_DW_args *)p, &a);
    ptl_internal_set_status(ptl_conv_dw_fp32_ig_batched(&a, 1));
}

static void dw16_from_kernel_args(const struct kernel_DW_args_fp16 *k, struct DepthWise_Conv_args_fp16 *a) {
    a->input = k->input;
    a->coeff = k->weights;
    a->output = k->output;
    a->Lpad = a->Rpad = a->Upad = a->Dpad = 0;
    a->skip_wg_grad = 0;
    a->skip_in_grad = 0;
    a->HWC = 0;
}

void dw_kernel_forward_fp16(void *p) {
    struct DepthWise_Conv_args_fp16 a;
    if (!p) { ptl_internal_set_status(1); return; }
    dw16_from_kernel_args((const struct kernel_DW_args_fp16 *)p, &a);
    ptl_internal_set_status(ptl_conv_dw_fp16_fw_batched(&a, 1));
}

void dw_kernel_weight_grad_fp16(void *p) {
    struct DepthWise_Conv_args_fp16 a;
    if (!p) { ptl_internal_set_status(1); return; }
    dw16_from_kernel_args((const struct kernel_DW_args_fp16 *)p, &a);
    ptl_internal_set_status(ptl_conv_dw_fp16_wg_batched(&a, 1));
}

void dw_kernel_input_grad_fp16(void *p) {
    struct DepthWise_Conv_args_fp16 a;
    if (!p) { ptl_internal_set_status(1); return; }
    dw16_from_kernel_args((const struct kernel_DW_args_fp16 *)p, &a);
    ptl_internal_set_status(ptl_conv_dw_fp16_ig_batched(&a, 1));
}

/* ---- Linear (lib/sources/pulp_linear_fp32.c, pulp_linear_fp16.c) ----------- */

void pulp_linear_fp32_fw_cl(void *p) { ptl_internal_set_status(ptl_linear_fp32_fw_batched(p, 1)); }
void pulp_linear_fp32_bw_param_grads_cl(void *p) { ptl_internal_set_status(ptl_linear_fp32_wg_batched(p, 1)); }
void pulp_linear_fp32_bw_input_grads_cl(void *p) { ptl_internal_set_status(ptl_linear_fp32_ig_batched(p, 1)); }

void pulp_linear_fp32_bw_cl(void *p) {
    struct Linear_args *a = (struct Linear_args *)p;
    int rc = 0;
    if (a && a->skip_wg_grad == 0) rc = ptl_linear_fp32_wg_batched(a, 1);
    if (a && a->skip_in_grad == 0) {
        int r2 = ptl_linear_fp32_ig_batched(a, 1);
        if (rc == 0) rc = r2;
    }
    ptl_internal_set_status(a ? rc : 1);
}

void pulp_linear_fp16_fw_cl(void *p) { ptl_internal_set_status(ptl_linear_fp16_fw_batched(p, 1)); }
void pulp_linear_fp16_bw_param_grads_cl(void *p) { ptl_internal_set_status(ptl_linear_fp16_wg_batched(p, 1)); }
void pulp_linear_fp16_bw_input_grads_cl(void *p) { ptl_internal_set_status(ptl_linear_fp16_ig_batched(p, 1)); }

void pulp_linear_fp16_bw_cl(void *p) {
    struct Linear_args_fp16 *a = (struct Linear_args_fp16 *)p;
    int rc = 0;
    if (a && a->skip_wg_grad == 0) rc = ptl_linear_fp16_wg_batched(a, 1);
    if (a && a->skip_in_grad == 0) {
        int r2 = ptl_linear_fp16_ig_batched(a, 1);
        if (rc == 0) rc = r2;
    }
    ptl_internal_set_status(a ? rc : 1);
}

/* ---- mm family and mm_manager ------------------------------------------------- */

static int mm32(const struct matMul_args *a) {
    if (!a) return 1;
    return ptl_mm_fp32(a->A, a->B, a->C, a->N, a->M, a->K, a->trans_B != 0);
}

static int mm16(const struct matMul_args_fp16 *a) {
    if (!a) return 1;
    return ptl_mm_fp16(a->A, a->B, a->C, a->N, a->M, a->K, a->trans_B != 0);
}

/* mm and mm_M differ only in which dimension the reference slices over its
 * cores (lib/sources/pulp_matmul_fp32.c:203-205 vs :359-361). */
void mm(void *p) { ptl_internal_set_status(mm32((const struct matMul_args *)p)); }
void mm_M(void *p) { ptl_internal_set_status(mm32((const struct matMul_args *)p)); }
void mm_fp16(void *p) { ptl_internal_set_status(mm16((const struct matMul_args_fp16 *)p)); }
void mm_M_fp16(void *p) { ptl_internal_set_status(mm16((const struct matMul_args_fp16 *)p)); }

/* The hand-unrolled variants (lib/include/pulp_matmul_fp32.h:72-244, pulp_matmul_fp16.h:56-107): the same
 * product as mm / mm_fp16, with loops unrolled over rows and columns for the cluster's cores and, in fp16,
 * two-element SIMD partial sums.  On the GPU they are one product, so every name lands on the same launcher;
 * the reference's harness calls them by name (tests/test_matmul/net.c:95-186). */
#define PTL_MM32_ALIAS(name) void name(void *p) { ptl_internal_set_status(mm32((const struct matMul_args *)p)); }
#define PTL_MM16_ALIAS(name) void name(void *p) { ptl_internal_set_status(mm16((const struct matMul_args_fp16 *)p)); }
PTL_MM32_ALIAS(mm_u2)
PTL_MM32_ALIAS(mm_unroll_1x2) PTL_MM32_ALIAS(mm_unroll_1x4) PTL_MM32_ALIAS(mm_unroll_1x8)
PTL_MM32_ALIAS(mm_unroll_2x1) PTL_MM32_ALIAS(mm_unroll_4x1) PTL_MM32_ALIAS(mm_unroll_8x1)
PTL_MM32_ALIAS(mm_unroll_2x2) PTL_MM32_ALIAS(mm_unroll_2x4) PTL_MM32_ALIAS(mm_unroll_4x2)
PTL_MM32_ALIAS(mm_unroll_4x4)
PTL_MM32_ALIAS(mm_M_u2)
PTL_MM32_ALIAS(mm_M_unroll_2x1) PTL_MM32_ALIAS(mm_M_unroll_4x1) PTL_MM32_ALIAS(mm_M_unroll_8x1)
PTL_MM32_ALIAS(mm_M_unroll_1x2) PTL_MM32_ALIAS(mm_M_unroll_1x4) PTL_MM32_ALIAS(mm_M_unroll_1x8)
PTL_MM32_ALIAS(mm_M_unroll_2x2) PTL_MM32_ALIAS(mm_M_unroll_4x2) PTL_MM32_ALIAS(mm_M_unroll_2x4)
PTL_MM32_ALIAS(mm_M_unroll_4x4)
PTL_MM16_ALIAS(mm_fp16_SIMD_2x4) PTL_MM16_ALIAS(mm_fp16_SIMD_4x8)
PTL_MM16_ALIAS(mm_fp16_unroll_8x1) PTL_MM16_ALIAS(mm_fp16_unroll_4x1) PTL_MM16_ALIAS(mm_fp16_unroll_2x1)
PTL_MM16_ALIAS(mm_M_fp16_SIMD_2x4) PTL_MM16_ALIAS(mm_M_fp16_SIMD_4x8)

/* Matrix x vector (lib/sources/pulp_matmul_fp16.c:1158-1176 and the 4x1 / 8x1 twins): C[i] = sum_k A[i*K+k] B[k].
 * With M > 1 the reference takes M as the vector's length when trans_B is set and stops otherwise ("second
 * tensor is not a vector", exit(1)); here that call is rejected with the same message and C is left alone. */
static int mv16(const struct matMul_args_fp16 *a) {
    if (!a) return 1;
    int K = a->K;
    if (a->M > 1) {
        if (!a->trans_B) {
            printf("\nError: second tensor is not a vector.\n");
            return 1;
        }
        K = a->M;
    }
    return ptl_mm_fp16(a->A, a->B, a->C, a->N, 1, K, 1);
}
void mv_fp16_SIMD_2x1(void *p) { ptl_internal_set_status(mv16((const struct matMul_args_fp16 *)p)); }
void mv_fp16_SIMD_4x1(void *p) { ptl_internal_set_status(mv16((const struct matMul_args_fp16 *)p)); }
void mv_fp16_SIMD_8x1(void *p) { ptl_internal_set_status(mv16((const struct matMul_args_fp16 *)p)); }

/* Selection checks of mm_manager (lib/sources/pulp_train_utils_fp32.c:1347-1669):
 * layer in {CONV2D, PW_CONV, LINEAR}, step in {FW, WGT_GRAD, IN_GRAD}, id within
 * the list.  Returns 0 when a matmul would have been selected. */
static int manager_select(int layer, int step, int id, int max_id) {
    if (layer != LAYER_CONV2D && layer != LAYER_PW_CONV && layer != LAYER_LINEAR) {
        printf("\nWrong layer_type selection!!\n");
        return 1;
    }
    if (step != STEP_FW && step != STEP_WGT_GRAD && step != STEP_IN_GRAD) {
        printf("\nWrong step selection!!\n");
        return 1;
    }
    if (id < 0 || id > max_id) {
        printf("\nWrong matmul selection!\n");
        return 1;
    }
    return 0;
}

void mm_manager(void *p) {
    struct mm_manager_args *m = (struct mm_manager_args *)p;
    int rc;
    if (!m || !m->mm_args) { ptl_internal_set_status(1); return; }
    rc = manager_select(m->layer_type, m->step_type, m->matmul_type, 23);
    if (rc == 0) rc = mm32(m->mm_args);
    /* bias epilogue of mm_manager (lib/sources/pulp_train_utils_fp32.c:1671-1682) */
    if (rc == 0 && m->mm_args->USE_BIASES == 1)
        rc = ptl_internal_bias_add_fp32(m->mm_args->C, m->mm_args->bias, m->mm_args->N, m->mm_args->M,
                                        m->mm_args->bias_transposed != 0);
    ptl_internal_set_status(rc);
}

void mm_manager_fp16(void *p) {
    struct mm_manager_args_fp16 *m = (struct mm_manager_args_fp16 *)p;
    int rc;
    if (!m || !m->mm_args) { ptl_internal_set_status(1); return; }
    rc = manager_select(m->layer_type, m->step_type, m->matmul_type, 8);
    if (rc == 0) rc = mm16(m->mm_args);
    if (rc == 0 && m->mm_args->USE_BIASES == 1)
        rc = ptl_internal_bias_add_fp16(m->mm_args->C, m->mm_args->bias, m->mm_args->N, m->mm_args->M,
                                        m->mm_args->bias_transposed != 0);
    ptl_internal_set_status(rc);
}

/* Product plus one per-output-channel bias add.  The reference adds the bias in
 * mm_manager and again here (lib/sources/pulp_conv2d_fp32.c:712-731); this adds
 * it once: CHW C[co][pix] += bias[co], HWC C[pix][co] += bias[co]. */
void im2col_conv2d_fw_kernel(void *p) {
    struct mm_manager_args *m = (struct mm_manager_args *)p;
    struct matMul_args *a;
    int rc;
    if (!m || !m->mm_args) { ptl_internal_set_status(1); return; }
    a = m->mm_args;
    rc = manager_select(m->layer_type, m->step_type, m->matmul_type, 23);
    if (rc == 0) rc = mm32(a);
    if (rc == 0 && a->USE_BIASES == 1) {
        if (a->HWC == 0)
            rc = ptl_internal_bias_add_fp32(a->C, a->bias, a->N, a->M, 1);
        else if (a->HWC == 1)
            rc = ptl_internal_bias_add_fp32(a->C, a->bias, a->N, a->M, 0);
        else
            printf("[im2col_conv2d_fw_kernel:] Invalid selection of the HWC layout (1 for HWC, 0 for CHW). Actual "
                   "value: %d. Biases not used, even if provided!\n", a->HWC);
    }
    ptl_internal_set_status(rc);
}

/* Product plus bias gradient = row sums of the output gradient, which is
 * operand A here (the reference sums operand C by mistake,
 * lib/sources/pulp_conv2d_fp32.c:752,795). */
void im2col_conv2d_param_grad_kernel(void *p) {
    struct mm_manager_args *m = (struct mm_manager_args *)p;
    struct matMul_args *a;
    int rc;
    if (!m || !m->mm_args) { ptl_internal_set_status(1); return; }
    a = m->mm_args;
    rc = manager_select(m->layer_type, m->step_type, m->matmul_type, 23);
    if (rc == 0) rc = mm32(a);
    if (rc == 0 && a->USE_BIASES == 1 && a->HWC == 0) rc = ptl_internal_rowsum_fp32(a->A, a->bias, a->N, a->K);
    ptl_internal_set_status(rc);
}

/* lib/sources/pulp_linear_fp32.c:199-232 */
void pulp_linear_fp32_fw_cl_kernel(void *p) { mm_manager(p); }

/* Product, then bias gradient = output gradient (lib/sources/pulp_linear_fp32.c:234-267). */
void pulp_linear_fp32_bw_param_grads_cl_kernel(void *p) {
    struct mm_manager_args *m = (struct mm_manager_args *)p;
    int use_bias, rc;
    if (!m || !m->mm_args) { ptl_internal_set_status(1); return; }
    /* the product itself takes no bias here */
    use_bias = m->mm_args->USE_BIASES;
    rc = manager_select(m->layer_type, m->step_type, m->matmul_type, 23);
    if (rc == 0) rc = mm32(m->mm_args);
    if (rc == 0 && use_bias == 1) {
        struct copy_args c;
        c.from = m->mm_args->A;
        c.to = m->mm_args->bias;
        c.size = m->mm_args->N;
        copy(&c);
        rc = ptl_last_status();
    }
    ptl_internal_set_status(rc);
}

/* ---- direct convolution kernels on matMul_args ------------------------------------
 * lib/sources/pulp_conv_naive_fp32.c:198 (A = input, B = weights, C = output),
 * :302 (A = input, B = weight gradient, C = output gradient),
 * :410 (A = input gradient, B = weights, C = output gradient);
 * H/W = input size, pH/pW = kernel size, pCin/pCout = channels. */

static void naive_setup32(const struct matMul_args *m, struct Conv2D_args *a, struct blob *in, struct blob *w,
                          struct blob *out, struct blob *bias) {
    int Ho = (m->H - m->pH + m->Upad + m->Dpad) / (m->stride_h > 0 ? m->stride_h : 1) + 1;
    int Wo = (m->W - m->pW + m->Lpad + m->Rpad) / (m->stride_w > 0 ? m->stride_w : 1) + 1;
    in->data = in->diff = NULL;
    in->C = m->pCin; in->H = m->H; in->W = m->W; in->dim = m->pCin * m->H * m->W;
    w->data = w->diff = NULL;
    w->C = m->pCin; w->H = m->pH; w->W = m->pW; w->dim = m->pCout * m->pCin * m->pH * m->pW;
    out->data = out->diff = NULL;
    out->C = m->pCout; out->H = Ho; out->W = Wo; out->dim = m->pCout * Ho * Wo;
    bias->data = bias->diff = m->bias;
    bias->C = bias->H = 1; bias->W = bias->dim = m->pCout;
    a->input = in; a->coeff = w; a->bias = bias; a->output = out;
    a->Lpad = m->Lpad; a->Rpad = m->Rpad; a->Upad = m->Upad; a->Dpad = m->Dpad;
    a->stride_h = m->stride_h; a->stride_w = m->stride_w;
    a->i2c_buffer = NULL; a->bt_buffer = NULL;
    a->skip_wg_grad = 0; a->skip_in_grad = 0; a->HWC = 0;
    a->opt_matmul_type_fw = a->opt_matmul_type_wg = a->opt_matmul_type_ig = 0;
    a->USE_BIASES = (m->USE_BIASES == 1 && m->bias) ? 1 : 0;
    a->USE_IM2COL = 0; a->USE_DMA_IM2COL = 0;
}

void naive_conv2d_fw_kernel_CHW(void *p) {
    struct matMul_args *m = (struct matMul_args *)p;
    struct Conv2D_args a; struct blob in, w, out, bias;
    if (!m) { ptl_internal_set_status(1); return; }
    naive_setup32(m, &a, &in, &w, &out, &bias);
    in.data = m->A; w.data = m->B; out.data = m->C;
    ptl_internal_set_status(ptl_conv2d_fp32_fw_batched(&a, 1));
}

void naive_conv2d_param_grad_kernel_CHW(void *p) {
    struct matMul_args *m = (struct matMul_args *)p;
    struct Conv2D_args a; struct blob in, w, out, bias;
    if (!m) { ptl_internal_set_status(1); return; }
    naive_setup32(m, &a, &in, &w, &out, &bias);
    in.data = m->A; w.diff = m->B; out.diff = m->C;
    ptl_internal_set_status(ptl_conv2d_fp32_wg_batched(&a, 1));
}

void naive_conv2d_in_grad_kernel_CHW(void *p) {
    struct matMul_args *m = (struct matMul_args *)p;
    struct Conv2D_args a; struct blob in, w, out, bias;
    if (!m) { ptl_internal_set_status(1); return; }
    naive_setup32(m, &a, &in, &w, &out, &bias);
    in.diff = m->A; w.data = m->B; out.diff = m->C;
    ptl_internal_set_status(ptl_conv2d_fp32_ig_batched(&a, 1));
}

static void naive_setup16(const struct matMul_args_fp16 *m, struct Conv2D_args_fp16 *a, struct blob_fp16 *in,
                          struct blob_fp16 *w, struct blob_fp16 *out, struct blob_fp16 *bias) {
    int Ho = (m->H - m->pH + m->Upad + m->Dpad) / (m->stride_h > 0 ? m->stride_h : 1) + 1;
    int Wo = (m->W - m->pW + m->Lpad + m->Rpad) / (m->stride_w > 0 ? m->stride_w : 1) + 1;
    in->data = in->diff = NULL;
    in->C = m->pCin; in->H = m->H; in->W = m->W; in->dim = m->pCin * m->H * m->W;
    w->data = w->diff = NULL;
    w->C = m->pCin; w->H = m->pH; w->W = m->pW; w->dim = m->pCout * m->pCin * m->pH * m->pW;
    out->data = out->diff = NULL;
    out->C = m->pCout; out->H = Ho; out->W = Wo; out->dim = m->pCout * Ho * Wo;
    bias->data = bias->diff = m->bias;
    bias->C = bias->H = 1; bias->W = bias->dim = m->pCout;
    a->input = in; a->coeff = w; a->bias = bias; a->output = out;
    a->Lpad = m->Lpad; a->Rpad = m->Rpad; a->Upad = m->Upad; a->Dpad = m->Dpad;
    a->stride_h = m->stride_h; a->stride_w = m->stride_w;
    a->i2c_buffer = NULL; a->bt_buffer = NULL;
    a->skip_wg_grad = 0; a->skip_in_grad = 0; a->HWC = 0;
    a->opt_matmul_type_fw = a->opt_matmul_type_wg = a->opt_matmul_type_ig = 0;
    a->USE_BIASES = (m->USE_BIASES == 1 && m->bias) ? 1 : 0;
    a->USE_IM2COL = 0; a->USE_DMA_IM2COL = 0;
}

void naive_conv2d_fw_kernel_CHW_fp16(void *p) {
    struct matMul_args_fp16 *m = (struct matMul_args_fp16 *)p;
    struct Conv2D_args_fp16 a; struct blob_fp16 in, w, out, bias;
    if (!m) { ptl_internal_set_status(1); return; }
    naive_setup16(m, &a, &in, &w, &out, &bias);
    in.data = m->A; w.data = m->B; out.data = m->C;
    ptl_internal_set_status(ptl_conv2d_fp16_fw_batched(&a, 1));
}

void naive_conv2d_param_grad_kernel_CHW_fp16(void *p) {
    struct matMul_args_fp16 *m = (struct matMul_args_fp16 *)p;
    struct Conv2D_args_fp16 a; struct blob_fp16 in, w, out, bias;
    if (!m) { ptl_internal_set_status(1); return; }
    naive_setup16(m, &a, &in, &w, &out, &bias);
    in.data = m->A; w.diff = m->B; out.diff = m->C;
    ptl_internal_set_status(ptl_conv2d_fp16_wg_batched(&a, 1));
}

void naive_conv2d_in_grad_kernel_CHW_fp16(void *p) {
    struct matMul_args_fp16 *m = (struct matMul_args_fp16 *)p;
    struct Conv2D_args_fp16 a; struct blob_fp16 in, w, out, bias;
    if (!m) { ptl_internal_set_status(1); return; }
    naive_setup16(m, &a, &in, &w, &out, &bias);
    in.diff = m->A; w.data = m->B; out.diff = m->C;
    ptl_internal_set_status(ptl_conv2d_fp16_ig_batched(&a, 1));
}

/* Fixed-geometry variants: 3x3 or 5x5 filter, stride 2, one row / column of padding on every side
 * (lib/sources/pulp_conv_naive_fp32.c:520, :581, :643, :702, :762, :825; pulp_conv_naive_fp16.c:471-756).
 * They read only H, W, pCin, pCout, the pointers and the bias fields of the struct; the geometry is in the name. */
#define PTL_FIXED_GEOMETRY(NAME, GENERIC, STRUCT, KSIZE)                                   \
    void NAME(void *p) {                                                                   \
        struct STRUCT m;                                                                   \
        if (!p) { ptl_internal_set_status(1); return; }                                    \
        m = *(const struct STRUCT *)p;                                                     \
        m.pH = m.pW = (KSIZE);                                                             \
        m.stride_h = m.stride_w = 2;                                                       \
        m.Lpad = m.Rpad = m.Upad = m.Dpad = 1;                                             \
        GENERIC(&m);                                                                       \
    }

PTL_FIXED_GEOMETRY(naive_conv2d_fw_kernel_CHW_k3x3_s2_p1, naive_conv2d_fw_kernel_CHW, matMul_args, 3)
PTL_FIXED_GEOMETRY(naive_conv2d_param_grad_kernel_CHW_k3x3_s2_p1, naive_conv2d_param_grad_kernel_CHW, matMul_args, 3)
PTL_FIXED_GEOMETRY(naive_conv2d_in_grad_kernel_CHW_k3x3_s2_p1, naive_conv2d_in_grad_kernel_CHW, matMul_args, 3)
PTL_FIXED_GEOMETRY(naive_conv2d_fw_kernel_CHW_k5x5_s2_p1, naive_conv2d_fw_kernel_CHW, matMul_args, 5)
PTL_FIXED_GEOMETRY(naive_conv2d_param_grad_kernel_CHW_k5x5_s2_p1, naive_conv2d_param_grad_kernel_CHW, matMul_args, 5)
PTL_FIXED_GEOMETRY(naive_conv2d_in_grad_kernel_CHW_k5x5_s2_p1, naive_conv2d_in_grad_kernel_CHW, matMul_args, 5)
PTL_FIXED_GEOMETRY(naive_conv2d_fw_kernel_CHW_k3x3_s2_p1_fp16, naive_conv2d_fw_kernel_CHW_fp16, matMul_args_fp16, 3)
PTL_FIXED_GEOMETRY(naive_conv2d_param_grad_kernel_CHW_k3x3_s2_p1_fp16, naive_conv2d_param_grad_kernel_CHW_fp16,
                   matMul_args_fp16, 3)
PTL_FIXED_GEOMETRY(naive_conv2d_in_grad_kernel_CHW_k3x3_s2_p1_fp16, naive_conv2d_in_grad_kernel_CHW_fp16,
                   matMul_args_fp16, 3)
PTL_FIXED_GEOMETRY(naive_conv2d_fw_kernel_CHW_k5x5_s2_p1_fp16, naive_conv2d_fw_kernel_CHW_fp16, matMul_args_fp16, 5)
PTL_FIXED_GEOMETRY(naive_conv2d_param_grad_kernel_CHW_k5x5_s2_p1_fp16, naive_conv2d_param_grad_kernel_CHW_fp16,
                   matMul_args_fp16, 5)
PTL_FIXED_GEOMETRY(naive_conv2d_in_grad_kernel_CHW_k5x5_s2_p1_fp16, naive_conv2d_in_grad_kernel_CHW_fp16,
                   matMul_args_fp16, 5)

/* Bias add on a row-major H x W matrix: t == 0 adds bias[column], otherwise bias[row]
 * (lib/sources/pulp_train_utils_fp32.c:1286-1324, pulp_train_utils_fp16.c twin). */
void mm_bias_add_transposed(void *p) {
    struct mm_bias_add_args *a = (struct mm_bias_add_args *)p;
    if (!a) { ptl_internal_set_status(1); return; }
    ptl_internal_set_status(ptl_internal_bias_add_fp32(a->mat, a->bias, a->H, a->W, a->t != 0));
}

void mm_bias_add_transposed_fp16(void *p) {
    struct mm_bias_add_args_fp16 *a = (struct mm_bias_add_args_fp16 *)p;
    if (!a) { ptl_internal_set_status(1); return; }
    ptl_internal_set_status(ptl_internal_bias_add_fp16(a->mat, a->bias, a->H, a->W, a->t != 0));
}

/* ---- Multi-head self-attention (lib/sources/pulp_mhsa_fp32.c:20, :648) and the row softmax
 * (lib/sources/pulp_act_fp32.c:187, :335) ------------------------------------------------- */

void pulp_mhsa_fp32_fw_cl(void *p) { ptl_internal_set_status(ptl_mhsa_fp32_fw_batched(p, 1)); }
void pulp_mhsa_fp32_bw_cl(void *p) { ptl_internal_set_status(ptl_mhsa_fp32_bw_batched(p, 1)); }
void pulp_softmax_fp32_fw_cl(void *p) { ptl_internal_set_status(ptl_internal_softmax_fp32(p, 0)); }
void pulp_softmax_fp32_bw_cl(void *p) { ptl_internal_set_status(ptl_internal_softmax_fp32(p, 1)); }

/* ---- Layers around the matmul core (lib/sources/pulp_act_fp32.c:83-129, pulp_residual_fp32.c:26-113,
 * pulp_pooling_fp32.c:24-122, pulp_losses_fp32.c:26-138, pulp_optimizers_fp32.c:26, pulp_batchnorm_fp32.c:28
 * and their fp16 twins) --------------------------------------------------------------------------- */

void pulp_relu_fp32_fw_cl(void *p) { ptl_internal_set_status(ptl_relu_fp32_batched(p, 1, 0)); }
void pulp_relu_fp32_bw_cl(void *p) { ptl_internal_set_status(ptl_relu_fp32_batched(p, 1, 1)); }
void relu_core_fw_fp32(void *p) { ptl_internal_set_status(ptl_relu_fp32_batched(p, 1, 0)); }
void relu_core_bw_fp32(void *p) { ptl_internal_set_status(ptl_relu_fp32_batched(p, 1, 1)); }
void pulp_relu_fp16_fw_cl(void *p) { ptl_internal_set_status(ptl_relu_fp16_batched(p, 1, 0)); }
void pulp_relu_fp16_bw_cl(void *p) { ptl_internal_set_status(ptl_relu_fp16_batched(p, 1, 1)); }
void relu_core_fw_fp16(void *p) { ptl_internal_set_status(ptl_relu_fp16_batched(p, 1, 0)); }
void relu_core_bw_fp16(void *p) { ptl_internal_set_status(ptl_relu_fp16_batched(p, 1, 1)); }

void pulp_residualconn_fp32_fw(void *p) { ptl_internal_set_status(ptl_residual_fp32_batched(p, 1, 0)); }
void pulp_sumnode_fp32_bw(void *p) { ptl_internal_set_status(ptl_residual_fp32_batched(p, 1, 1)); }
void pulp_residualconn_fp32_bw(void *p) { ptl_internal_set_status(ptl_residual_fp32_batched(p, 1, 2)); }
void pulp_residualconn_fp16_fw(void *p) { ptl_internal_set_status(ptl_residual_fp16_batched(p, 1, 0)); }
void pulp_sumnode_fp16_bw(void *p) { ptl_internal_set_status(ptl_residual_fp16_batched(p, 1, 1)); }
void pulp_residualconn_fp16_bw(void *p) { ptl_internal_set_status(ptl_residual_fp16_batched(p, 1, 2)); }

void pulp_avgpool_fp32_fw_cl(void *p) { ptl_internal_set_status(ptl_avgpool_fp32_batched(p, 1, 0)); }
void pulp_avgpool_fp32_bw_cl(void *p) { ptl_internal_set_status(ptl_avgpool_fp32_batched(p, 1, 1)); }
void pulp_avgpool_fp16_fw_cl(void *p) { ptl_internal_set_status(ptl_avgpool_fp16_batched(p, 1, 0)); }
void pulp_avgpool_fp16_bw_cl(void *p) { ptl_internal_set_status(ptl_avgpool_fp16_batched(p, 1, 1)); }

void pulp_CrossEntropyLoss(void *p) { ptl_internal_set_status(ptl_cross_entropy_fp32_batched(p, 1, 0)); }
void pulp_CrossEntropyLoss_backward(void *p) { ptl_internal_set_status(ptl_cross_entropy_fp32_batched(p, 1, 1)); }
void pulp_CrossEntropyLoss_fp16(void *p) { ptl_internal_set_status(ptl_cross_entropy_fp16_batched(p, 1, 0)); }
void pulp_CrossEntropyLoss_backward_fp16(void *p) { ptl_internal_set_status(ptl_cross_entropy_fp16_batched(p, 1, 1)); }

void pulp_gradient_descent_fp32(void *p) { ptl_internal_set_status(ptl_gradient_descent_fp32(p)); }
void pulp_gradient_descent_fp16(void *p) { ptl_internal_set_status(ptl_gradient_descent_fp16(p)); }

void pulp_batch_norm_fp32_fw_cl(void *p) { ptl_internal_set_status(ptl_batch_norm_fp32_fw(p)); }
void pulp_batch_norm_parallelized_fp32_fw_cl(void *p) { ptl_internal_set_status(ptl_batch_norm_fp32_fw(p)); }
