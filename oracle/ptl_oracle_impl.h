/*
 * TEST INFRASTRUCTURE - type-generic body of the CPU oracle.
 *
 * Included twice by ptl_oracle.c, once per data type.  The including file
 * defines:
 *   T            element type (float or _Float16)
 *   MAC(acc,a,b) one multiply-accumulate step in the reference's arithmetic
 *   NAME(x)      x##_fp32 or x##_fp16
 *   BLOB, MM_ARGS, CONV_ARGS, PW_ARGS, DW_ARGS, LIN_ARGS, I2C_ARGS, BT_ARGS,
 *   TR_ARGS, LAY_ARGS, PAD_ARGS   the argument structs of that type
 *   DW_SH(a), DW_SW(a)            depthwise strides (the fp16 struct has none)
 *   PW_HWC_W_CI_MAJOR             1 if HWC pointwise weights are [Ci][Co]
 *
 * Every function states the reference code it restates.  Loops keep the
 * reference's summation order (k innermost, sequential accumulator of type
 * T), so fp16 results carry the reference's own fp16 rounding.
 */

/* ---- mm: lib/sources/pulp_matmul_fp32.c:190-264 (mm), :345-398 (mm_M);
 *          lib/sources/pulp_matmul_fp16.c:191-270 (mm_fp16).
 * C[i*M+j] = sum_k A[i*K+k] * B[k*M+j]   (trans_B == 0)
 *            sum_k A[i*K+k] * B[j*K+k]   (trans_B != 0)
 * K == 1 is a plain product; K == 0 leaves C untouched.  The j loop is blocked
 * by 8 only to give the compiler independent accumulators; each output still
 * sums its k terms in increasing k order. */
static void NAME(mm_core)(const T *A, const T *B, T *C, int N, int M, int K, int trans_B) {
    if (K <= 0) return;
#pragma omp parallel for schedule(static)
    for (int i = 0; i < N; i++) {
        for (int j0 = 0; j0 < M; j0 += 8) {
            int jn = M - j0 < 8 ? M - j0 : 8;
            T acc[8];
            for (int jj = 0; jj < jn; jj++) acc[jj] = (T)0;
            if (K == 1) {
                for (int jj = 0; jj < jn; jj++) C[i * M + j0 + jj] = A[i] * B[j0 + jj];
                continue;
            }
            if (!trans_B) {
                for (int k = 0; k < K; k++) {
                    T a = A[(size_t)i * K + k];
                    const T *b = B + (size_t)k * M + j0;
                    for (int jj = 0; jj < jn; jj++) MAC(acc[jj], a, b[jj]);
                }
            } else {
                for (int jj = 0; jj < jn; jj++) {
                    const T *b = B + (size_t)(j0 + jj) * K;
                    T s = (T)0;
                    for (int k = 0; k < K; k++) MAC(s, A[(size_t)i * K + k], b[k]);
                    acc[jj] = s;
                }
            }
            for (int jj = 0; jj < jn; jj++) C[(size_t)i * M + j0 + jj] = acc[jj];
        }
    }
}

void NAME(orc_mm)(void *p) {
    MM_ARGS *a = (MM_ARGS *)p;
    NAME(mm_core)(a->A, a->B, a->C, a->N, a->M, a->K, a->trans_B);
}

/* ---- im2row / im2col: lib/sources/pulp_im2col_fp32.c:29-232 (CHW), :430-546
 * (HWC), :668-1012 (column-major twin); fp16: pulp_im2col_fp16.c:29, :526.
 * Patch matrix entry (p, q): p = patch position, q = position inside the
 * receptive field ordered (c,hk,wk) for CHW and (hk,wk,c) for HWC.
 *   mod 0: p = ho*Wt+wo, value = in[c, ho*sh-Up+hk, wo*sw-Lp+wk]
 *   mod 1: p = hi*Wi+wi, value = outdiff[c, hi-(Hk-1)+hk, wi-(Wk-1)+wk]
 * zero outside the tensor.  The reference tests the padded border with
 * h > Ho+Hk-Dpad (pulp_im2col_fp32.c:175), which equals the true bound only
 * for Up+Dp == 2; the true bound is used.  im2row stores buf[p*Q+q], im2col
 * buf[q*P+p]. */
static void NAME(patch_build)(const I2C_ARGS *a, int col_major) {
    int Lp = (uint8_t)a->Lpad, Rp = (uint8_t)a->Rpad, Up = (uint8_t)a->Upad, Dp = (uint8_t)a->Dpad;
    int mod = (uint8_t)a->mod, sh = (uint8_t)a->stride_h, sw = (uint8_t)a->stride_w, hwc = (uint8_t)a->HWC;
    int Hin = a->input->H, Win = a->input->W, Cin = a->input->C;
    int Hk = a->c->H, Wk = a->c->W, Co = a->output->C;
    int C, Hs, Ws, Hp, Wp, hmul, hadd, wmul, wadd;
    const T *src;
    if (mod == 0) {
        if (sh == 0 || sw == 0) return;
        if ((Hin - Hk + Up + Dp + sh) % sh > 0 || (Win - Wk + Lp + Rp + sw) % sw > 0) return;
        C = Cin; Hs = Hin; Ws = Win;
        Hp = (Hin - Hk + Up + Dp + sh) / sh;
        Wp = (Win - Wk + Lp + Rp + sw) / sw;
        hmul = sh; hadd = -Up; wmul = sw; wadd = -Lp;
        src = a->input->data;
    } else {
        C = Co; Hs = a->output->H; Ws = a->output->W;
        Hp = Hin; Wp = Win;
        hmul = 1; hadd = -(Hk - 1); wmul = 1; wadd = -(Wk - 1);
        src = a->output->diff;
    }
    int Q = C * Hk * Wk, P = Hp * Wp;
#pragma omp parallel for schedule(static)
    for (int p = 0; p < P; p++) {
        int hp = p / Wp, wp = p % Wp;
        for (int c = 0; c < C; c++)
            for (int hk = 0; hk < Hk; hk++)
                for (int wk = 0; wk < Wk; wk++) {
                    int q = hwc ? (hk * Wk + wk) * C + c : (c * Hk + hk) * Wk + wk;
                    int h = hp * hmul + hadd + hk, w = wp * wmul + wadd + wk;
                    T v = (T)0;
                    if (h >= 0 && h < Hs && w >= 0 && w < Ws)
                        v = hwc ? src[((size_t)h * Ws + w) * C + c] : src[((size_t)c * Hs + h) * Ws + w];
                    if (col_major)
                        a->pBuffer[(size_t)q * P + p] = v;
                    else
                        a->pBuffer[(size_t)p * Q + q] = v;
                }
    }
}

void NAME(orc_im2row)(void *p) { NAME(patch_build)((const I2C_ARGS *)p, 0); }
void NAME(orc_im2col)(void *p) { NAME(patch_build)((const I2C_ARGS *)p, 1); }

/* ---- blocktranspose: lib/sources/pulp_im2col_fp32.c:1020-1072.
 * CHW: bt[c*Co*HW + k*HW + i] = w[k*Ci*HW + c*HW + (HW-1-i)]
 * HWC: bt[ci*Hk*Wk*Co + hk*Wk*Co + wk*Co + co] = w[co*Hk*Wk*Ci + (Hk-1-hk)*Wk*Ci + (Wk-1-wk)*Ci + ci] */
void NAME(orc_blocktransp)(void *p) {
    BT_ARGS *a = (BT_ARGS *)p;
    int Ci = a->Cin, Co = a->Cout, Hk = a->Hk, Wk = a->Wk, HW = Hk * Wk;
    if ((uint8_t)a->HWC == 0) {
        for (int k = 0; k < Co; k++)
            for (int c = 0; c < Ci; c++)
                for (int i = 0; i < HW; i++)
                    a->bt_weights[i + k * HW + c * Co * HW] = a->weights[(HW - 1 - i) + c * HW + k * Ci * HW];
    } else if ((uint8_t)a->HWC == 1) {
        for (int co = 0; co < Co; co++)
            for (int hk = 0; hk < Hk; hk++)
                for (int wk = 0; wk < Wk; wk++)
                    for (int ci = 0; ci < Ci; ci++)
                        a->bt_weights[ci * HW * Co + wk * Co + hk * Wk * Co + co] =
                            a->weights[ci + (Wk - 1 - wk) * Ci + (Hk - 1 - hk) * Wk * Ci + co * HW * Ci];
    }
}

/* ---- direct Conv2D: lib/sources/pulp_conv_naive_fp32.c:198-300 (forward),
 * :302-408 (weight gradient), :410-518 (input gradient); fp16 twins in
 * pulp_conv_naive_fp16.c.  Full stride and padding; loop order and summation
 * order of the reference (ci, hk, wk innermost for forward; ho, wo innermost
 * for the weight gradient; co, hk, wk for the input gradient).  Layout-aware
 * accessors extend the same loops to HWC tensors (weights [co][hk][wk][ci]). */
#define IDX_ACT(hwc, C, H, W, c, h, w) \
    ((hwc) ? (((size_t)(h) * (W) + (w)) * (C) + (c)) : (((size_t)(c) * (H) + (h)) * (W) + (w)))
#define IDX_WGT(hwc, Ci, Hk, Wk, co, ci, hk, wk)                          \
    ((hwc) ? ((((size_t)(co) * (Hk) + (hk)) * (Wk) + (wk)) * (Ci) + (ci)) \
           : ((((size_t)(co) * (Ci) + (ci)) * (Hk) + (hk)) * (Wk) + (wk)))

static void NAME(conv_fw_one)(const T *X, const T *Wt, const T *bias, T *Y, int Ci, int H, int W, int Co, int Hk,
                              int Wk, int sh, int sw, int Up, int Dp, int Lp, int Rp, int hwc) {
    int Ho = (H - Hk + Up + Dp) / sh + 1, Wo = (W - Wk + Lp + Rp) / sw + 1;
#pragma omp parallel for schedule(static)
    for (int co = 0; co < Co; co++)
        for (int ho = 0; ho < Ho; ho++)
            for (int wo = 0; wo < Wo; wo++) {
                T temp = (T)0;
                for (int ci = 0; ci < Ci; ci++)
                    for (int hk = 0; hk < Hk; hk++)
                        for (int wk = 0; wk < Wk; wk++) {
                            int h = sh * ho + hk - Up, w = sw * wo + wk - Lp;
                            if (h >= 0 && w >= 0 && h < H && w < W)
                                MAC(temp, X[IDX_ACT(hwc, Ci, H, W, ci, h, w)],
                                    Wt[IDX_WGT(hwc, Ci, Hk, Wk, co, ci, hk, wk)]);
                        }
                if (bias) temp = temp + bias[co];
                Y[IDX_ACT(hwc, Co, Ho, Wo, co, ho, wo)] = temp;
            }
}

static void NAME(conv_wg_one)(const T *X, const T *dY, T *dW, T *db, int Ci, int H, int W, int Co, int Hk, int Wk,
                              int sh, int sw, int Up, int Dp, int Lp, int Rp, int hwc) {
    int Ho = (H - Hk + Up + Dp) / sh + 1, Wo = (W - Wk + Lp + Rp) / sw + 1;
#pragma omp parallel for schedule(static)
    for (int co = 0; co < Co; co++) {
        for (int hk = 0; hk < Hk; hk++)
            for (int wk = 0; wk < Wk; wk++)
                for (int ci = 0; ci < Ci; ci++) {
                    T temp = (T)0;
                    for (int ho = 0; ho < Ho; ho++)
                        for (int wo = 0; wo < Wo; wo++) {
                            int h = sh * ho + hk - Up, w = sw * wo + wk - Lp;
                            if (h >= 0 && w >= 0 && h < H && w < W)
                                MAC(temp, dY[IDX_ACT(hwc, Co, Ho, Wo, co, ho, wo)],
                                    X[IDX_ACT(hwc, Ci, H, W, ci, h, w)]);
                        }
                    dW[IDX_WGT(hwc, Ci, Hk, Wk, co, ci, hk, wk)] = temp;
                }
        if (db) {
            T s = (T)0;
            for (int ho = 0; ho < Ho; ho++)
                for (int wo = 0; wo < Wo; wo++) s = s + dY[IDX_ACT(hwc, Co, Ho, Wo, co, ho, wo)];
            db[co] = s;
        }
    }
}

static void NAME(conv_ig_one)(const T *Wt, const T *dY, T *dX, int Ci, int H, int W, int Co, int Hk, int Wk, int sh,
                              int sw, int Up, int Dp, int Lp, int Rp, int hwc) {
    int Ho = (H - Hk + Up + Dp) / sh + 1, Wo = (W - Wk + Lp + Rp) / sw + 1;
#pragma omp parallel for schedule(static)
    for (int ci = 0; ci < Ci; ci++)
        for (int hi = 0; hi < H; hi++)
            for (int wi = 0; wi < W; wi++) {
                T temp = (T)0;
                /* the reference walks the flipped kernel: tap (Hk-1-hk', Wk-1-wk')
                 * meets output row (hi + hk' - (Hk-1-Up)) / sh */
                for (int co = 0; co < Co; co++)
                    for (int hk = 0; hk < Hk; hk++)
                        for (int wk = 0; wk < Wk; wk++) {
                            int hq = hi + hk - (Hk - 1 - Up), wq = wi + wk - (Wk - 1 - Lp);
                            if (hq < 0 || wq < 0 || hq % sh != 0 || wq % sw != 0) continue;
                            int ho = hq / sh, wo = wq / sw;
                            if (ho >= Ho || wo >= Wo) continue;
                            MAC(temp, Wt[IDX_WGT(hwc, Ci, Hk, Wk, co, ci, Hk - 1 - hk, Wk - 1 - wk)],
                                dY[IDX_ACT(hwc, Co, Ho, Wo, co, ho, wo)]);
                        }
                dX[IDX_ACT(hwc, Ci, H, W, ci, hi, wi)] = temp;
            }
}

/* Layer entry points, lib/sources/pulp_conv2d_fp32.c:27 / :240 / :454 (fp16:
 * pulp_conv2d_fp16.c).  Both USE_IM2COL settings give the direct-kernel
 * result: the im2col route equals it wherever the reference defines it (no
 * padding; forward also with padding) and is undefined elsewhere because its
 * weight/input-gradient im2row is called with the pads forced to zero
 * (pulp_conv2d_fp32.c:298-301, :508-513).  Samples are stored back to back;
 * the weight gradient is the fp32 sum of the per-sample gradients, rounded to
 * T once. */
void NAME(orc_conv2d_fw)(const CONV_ARGS *a, int ns) {
    int Ci = a->input->C, H = a->input->H, W = a->input->W, Co = a->output->C, Hk = a->coeff->H, Wk = a->coeff->W;
    int Ho = a->output->H, Wo = a->output->W;
    for (int n = 0; n < ns; n++)
        NAME(conv_fw_one)(a->input->data + (size_t)n * Ci * H * W, a->coeff->data,
                          a->USE_BIASES == 1 ? a->bias->data : NULL, a->output->data + (size_t)n * Co * Ho * Wo, Ci,
                          H, W, Co, Hk, Wk, a->stride_h, a->stride_w, a->Upad, a->Dpad, a->Lpad, a->Rpad, a->HWC);
}

void NAME(orc_conv2d_wg)(const CONV_ARGS *a, int ns) {
    int Ci = a->input->C, H = a->input->H, W = a->input->W, Co = a->output->C, Hk = a->coeff->H, Wk = a->coeff->W;
    int Ho = a->output->H, Wo = a->output->W;
    size_t wn = (size_t)Co * Ci * Hk * Wk;
    T *one = (T *)malloc(wn * sizeof(T));
    T *bone = (T *)malloc((size_t)Co * sizeof(T));
    float *sum = (float *)calloc(wn, sizeof(float));
    float *bsum = (float *)calloc((size_t)Co, sizeof(float));
    int bias = a->USE_BIASES == 1;
    for (int n = 0; n < ns; n++) {
        NAME(conv_wg_one)(a->input->data + (size_t)n * Ci * H * W, a->output->diff + (size_t)n * Co * Ho * Wo, one,
                          bias ? bone : NULL, Ci, H, W, Co, Hk, Wk, a->stride_h, a->stride_w, a->Upad, a->Dpad,
                          a->Lpad, a->Rpad, a->HWC);
        for (size_t i = 0; i < wn; i++) sum[i] += (float)one[i];
        if (bias)
            for (int i = 0; i < Co; i++) bsum[i] += (float)bone[i];
    }
    for (size_t i = 0; i < wn; i++) a->coeff->diff[i] = (T)sum[i];
    if (bias)
        for (int i = 0; i < Co; i++) a->bias->diff[i] = (T)bsum[i];
    free(one); free(bone); free(sum); free(bsum);
}

void NAME(orc_conv2d_ig)(const CONV_ARGS *a, int ns) {
    int Ci = a->input->C, H = a->input->H, W = a->input->W, Co = a->output->C, Hk = a->coeff->H, Wk = a->coeff->W;
    int Ho = a->output->H, Wo = a->output->W;
    for (int n = 0; n < ns; n++)
        NAME(conv_ig_one)(a->coeff->data, a->output->diff + (size_t)n * Co * Ho * Wo,
                          a->input->diff + (size_t)n * Ci * H * W, Ci, H, W, Co, Hk, Wk, a->stride_h, a->stride_w,
                          a->Upad, a->Dpad, a->Lpad, a->Rpad, a->HWC);
}

/* The im2col route of the CHW layer, literally: im2row into i2c_buffer, then
 * mm (forward: pulp_conv2d_fp32.c:71-113; weight gradient :294-333 with the
 * pads forced to 0; input gradient :504-548 with blocktranspose into
 * bt_buffer).  Defined for one sample; meaningful for the weight and input
 * gradient only when the layer has no padding and unit stride. */
void NAME(orc_conv2d_im2col_route)(const CONV_ARGS *a, int step) {
    int Ci = a->input->C, H = a->input->H, W = a->input->W, Co = a->output->C, Hk = a->coeff->H, Wk = a->coeff->W;
    int Ho = a->output->H, Wo = a->output->W;
    I2C_ARGS ia;
    ia.input = a->input; ia.c = a->coeff; ia.output = a->output; ia.pBuffer = a->i2c_buffer;
    ia.HWC = 0; ia.USE_DMA = 0;
    if (step == STEP_FW) {
        ia.Lpad = a->Lpad; ia.Rpad = a->Rpad; ia.Upad = a->Upad; ia.Dpad = a->Dpad;
        ia.mod = 0; ia.stride_w = a->stride_w; ia.stride_h = a->stride_h;
        NAME(patch_build)(&ia, 0);
        NAME(mm_core)(a->coeff->data, a->i2c_buffer, a->output->data, Co, Ho * Wo, Ci * Hk * Wk, 1);
    } else if (step == STEP_WGT_GRAD) {
        ia.Lpad = ia.Rpad = ia.Upad = ia.Dpad = 0;
        ia.mod = 0; ia.stride_w = a->stride_w; ia.stride_h = a->stride_h;
        NAME(patch_build)(&ia, 0);
        NAME(mm_core)(a->output->diff, a->i2c_buffer, a->coeff->diff, Co, Ci * Hk * Wk, Ho * Wo, 0);
    } else {
        ia.Lpad = ia.Rpad = ia.Upad = ia.Dpad = 0;
        ia.mod = 1; ia.stride_w = 1; ia.stride_h = 1;
        NAME(patch_build)(&ia, 0);
        BT_ARGS ba;
        ba.weights = a->coeff->data; ba.bt_weights = a->bt_buffer;
        ba.Cin = Ci; ba.Cout = Co; ba.Hk = Hk; ba.Wk = Wk; ba.HWC = 0;
        NAME(orc_blocktransp)(&ba);
        NAME(mm_core)(a->bt_buffer, a->i2c_buffer, a->input->diff, Ci, H * W, Co * Hk * Wk, 1);
    }
}

/* ---- pointwise: lib/sources/pulp_conv_pw_fp32.c:27-104, :121-231, :233-359;
 * fp16: pulp_conv_pw_fp16.c.  CHW: Y = W[Co x Ci] * X[Ci x HW];
 * dW = dY * X^T; dX = W^T * dY.  HWC: Y[HW x Co] = X[HW x Ci] * W; dW and dX
 * accordingly.  The fp32 input-gradient step of the reference transposes W
 * with rows and columns swapped (pulp_conv_pw_fp32.c:278-279), which is only
 * right for Ci == Co; the mathematically transposed W is used here, as the
 * fp16 layer does (pulp_conv_pw_fp16.c:293-294). */
static size_t NAME(pw_widx)(int hwc, int Ci, int Co, int co, int ci) {
    if (hwc && PW_HWC_W_CI_MAJOR) return (size_t)ci * Co + co;
    return (size_t)co * Ci + ci;
}

static void NAME(pw_fw_one)(const T *X, const T *Wt, T *Y, int Ci, int Co, int HW, int hwc) {
#pragma omp parallel for schedule(static)
    for (int co = 0; co < Co; co++)
        for (int p = 0; p < HW; p++) {
            T temp = (T)0;
            for (int ci = 0; ci < Ci; ci++)
                MAC(temp, Wt[NAME(pw_widx)(hwc, Ci, Co, co, ci)], hwc ? X[(size_t)p * Ci + ci] : X[(size_t)ci * HW + p]);
            if (hwc) Y[(size_t)p * Co + co] = temp; else Y[(size_t)co * HW + p] = temp;
        }
}

static void NAME(pw_wg_one)(const T *X, const T *dY, T *dW, int Ci, int Co, int HW, int hwc) {
#pragma omp parallel for schedule(static)
    for (int co = 0; co < Co; co++)
        for (int ci = 0; ci < Ci; ci++) {
            T temp = (T)0;
            for (int p = 0; p < HW; p++)
                MAC(temp, hwc ? dY[(size_t)p * Co + co] : dY[(size_t)co * HW + p],
                    hwc ? X[(size_t)p * Ci + ci] : X[(size_t)ci * HW + p]);
            dW[NAME(pw_widx)(hwc, Ci, Co, co, ci)] = temp;
        }
}

static void NAME(pw_ig_one)(const T *Wt, const T *dY, T *dX, int Ci, int Co, int HW, int hwc) {
#pragma omp parallel for schedule(static)
    for (int ci = 0; ci < Ci; ci++)
        for (int p = 0; p < HW; p++) {
            T temp = (T)0;
            for (int co = 0; co < Co; co++)
                MAC(temp, Wt[NAME(pw_widx)(hwc, Ci, Co, co, ci)], hwc ? dY[(size_t)p * Co + co] : dY[(size_t)co * HW + p]);
            if (hwc) dX[(size_t)p * Ci + ci] = temp; else dX[(size_t)ci * HW + p] = temp;
        }
}

void NAME(orc_conv_pw_fw)(const PW_ARGS *a, int ns) {
    int Ci = a->input->C, Co = a->output->C, HW = a->input->H * a->input->W;
    for (int n = 0; n < ns; n++)
        NAME(pw_fw_one)(a->input->data + (size_t)n * Ci * HW, a->coeff->data, a->output->data + (size_t)n * Co * HW,
                        Ci, Co, HW, a->HWC);
}

void NAME(orc_conv_pw_wg)(const PW_ARGS *a, int ns) {
    int Ci = a->input->C, Co = a->output->C, HW = a->input->H * a->input->W;
    size_t wn = (size_t)Co * Ci;
    T *one = (T *)malloc(wn * sizeof(T));
    float *sum = (float *)calloc(wn, sizeof(float));
    for (int n = 0; n < ns; n++) {
        NAME(pw_wg_one)(a->input->data + (size_t)n * Ci * HW, a->output->diff + (size_t)n * Co * HW, one, Ci, Co, HW,
                        a->HWC);
        for (size_t i = 0; i < wn; i++) sum[i] += (float)one[i];
    }
    for (size_t i = 0; i < wn; i++) a->coeff->diff[i] = (T)sum[i];
    free(one); free(sum);
}

void NAME(orc_conv_pw_ig)(const PW_ARGS *a, int ns) {
    int Ci = a->input->C, Co = a->output->C, HW = a->input->H * a->input->W;
    for (int n = 0; n < ns; n++)
        NAME(pw_ig_one)(a->coeff->data, a->output->diff + (size_t)n * Co * HW, a->input->diff + (size_t)n * Ci * HW,
                        Ci, Co, HW, a->HWC);
}

/* ---- depthwise: lib/sources/pulp_conv_naive_fp32.c:29-110 (forward with
 * stride and padding), :113-150 (weight gradient), :153-195 (input gradient);
 * fp16: pulp_conv_naive_fp16.c:32, :75, :118.  The reference's two gradient
 * kernels are written for unit stride and no padding; the loops below keep
 * their order and reduce to them in that case, and otherwise follow the
 * geometry of the forward. */
static void NAME(dw_fw_one)(const T *X, const T *Wt, T *Y, int C, int H, int W, int Hk, int Wk, int Ho, int Wo,
                            int sh, int sw, int Up, int Lp) {
#pragma omp parallel for schedule(static)
    for (int ch = 0; ch < C; ch++)
        for (int ho = 0; ho < Ho; ho++)
            for (int wo = 0; wo < Wo; wo++) {
                T temp = (T)0;
                for (int hk = 0; hk < Hk; hk++)
                    for (int wk = 0; wk < Wk; wk++) {
                        int h = sh * ho + hk - Up, w = sw * wo + wk - Lp;
                        if (h >= 0 && w >= 0 && h < H && w < W)
                            MAC(temp, Wt[wk + hk * Wk + ch * Hk * Wk], X[w + h * W + (size_t)ch * H * W]);
                    }
                Y[wo + ho * Wo + (size_t)ch * Ho * Wo] = temp;
            }
}

static void NAME(dw_wg_one)(const T *X, const T *dY, T *dW, int C, int H, int W, int Hk, int Wk, int Ho, int Wo,
                            int sh, int sw, int Up, int Lp) {
#pragma omp parallel for schedule(static)
    for (int ch = 0; ch < C; ch++)
        for (int hk = 0; hk < Hk; hk++)
            for (int wk = 0; wk < Wk; wk++) {
                T temp = (T)0;
                for (int ho = 0; ho < Ho; ho++)
                    for (int wo = 0; wo < Wo; wo++) {
                        int h = sh * ho + hk - Up, w = sw * wo + wk - Lp;
                        if (h >= 0 && w >= 0 && h < H && w < W)
                            MAC(temp, X[w + h * W + (size_t)ch * H * W], dY[wo + ho * Wo + (size_t)ch * Ho * Wo]);
                    }
                dW[wk + hk * Wk + ch * Hk * Wk] = temp;
            }
}

static void NAME(dw_ig_one)(const T *Wt, const T *dY, T *dX, int C, int H, int W, int Hk, int Wk, int Ho, int Wo,
                            int sh, int sw, int Up, int Lp) {
#pragma omp parallel for schedule(static)
    for (int ch = 0; ch < C; ch++)
        for (int hin = 0; hin < H; hin++)
            for (int win = 0; win < W; win++) {
                T temp = (T)0;
                for (int hk = 0; hk < Hk; hk++)
                    for (int wk = 0; wk < Wk; wk++) {
                        int hq = hin + hk - (Hk - 1 - Up), wq = win + wk - (Wk - 1 - Lp);
                        if (hq < 0 || wq < 0 || hq % sh != 0 || wq % sw != 0) continue;
                        int ho = hq / sh, wo = wq / sw;
                        if (ho >= Ho || wo >= Wo) continue;
                        MAC(temp, Wt[(Wk - 1 - wk) + (Hk - 1 - hk) * Wk + ch * Hk * Wk],
                            dY[wo + ho * Wo + (size_t)ch * Ho * Wo]);
                    }
                dX[win + hin * W + (size_t)ch * H * W] = temp;
            }
}

void NAME(orc_conv_dw_fw)(const DW_ARGS *a, int ns) {
    int C = a->input->C, H = a->input->H, W = a->input->W, Hk = a->coeff->H, Wk = a->coeff->W;
    int Ho = a->output->H, Wo = a->output->W;
    for (int n = 0; n < ns; n++)
        NAME(dw_fw_one)(a->input->data + (size_t)n * C * H * W, a->coeff->data,
                        a->output->data + (size_t)n * C * Ho * Wo, C, H, W, Hk, Wk, Ho, Wo, DW_SH(a), DW_SW(a),
                        a->Upad, a->Lpad);
}

void NAME(orc_conv_dw_wg)(const DW_ARGS *a, int ns) {
    int C = a->input->C, H = a->input->H, W = a->input->W, Hk = a->coeff->H, Wk = a->coeff->W;
    int Ho = a->output->H, Wo = a->output->W;
    size_t wn = (size_t)C * Hk * Wk;
    T *one = (T *)malloc(wn * sizeof(T));
    float *sum = (float *)calloc(wn, sizeof(float));
    for (int n = 0; n < ns; n++) {
        NAME(dw_wg_one)(a->input->data + (size_t)n * C * H * W, a->output->diff + (size_t)n * C * Ho * Wo, one, C, H,
                        W, Hk, Wk, Ho, Wo, DW_SH(a), DW_SW(a), a->Upad, a->Lpad);
        for (size_t i = 0; i < wn; i++) sum[i] += (float)one[i];
    }
    for (size_t i = 0; i < wn; i++) a->coeff->diff[i] = (T)sum[i];
    free(one); free(sum);
}

void NAME(orc_conv_dw_ig)(const DW_ARGS *a, int ns) {
    int C = a->input->C, H = a->input->H, W = a->input->W, Hk = a->coeff->H, Wk = a->coeff->W;
    int Ho = a->output->H, Wo = a->output->W;
    for (int n = 0; n < ns; n++)
        NAME(dw_ig_one)(a->coeff->data, a->output->diff + (size_t)n * C * Ho * Wo,
                        a->input->diff + (size_t)n * C * H * W, C, H, W, Hk, Wk, Ho, Wo, DW_SH(a), DW_SW(a), a->Upad,
                        a->Lpad);
}

/* ---- Linear: lib/sources/pulp_linear_fp32.c:25-65 (y = W x via mm, N=out,
 * K=in, M=1), :85-139 (dW = dy (x) x via mm with K=1; db = dy, :261-265),
 * :142-196 (dx = dy^T W via mm_M, N=1, K=out, M=in).  Bias: y += b as the fp16
 * layer does (pulp_linear_fp16.c:252-258). */
void NAME(orc_linear_fw)(const LIN_ARGS *a, int ns) {
    int in = a->input->dim, out = a->output->dim;
    for (int n = 0; n < ns; n++) {
        T *y = a->output->data + (size_t)n * out;
        NAME(mm_core)(a->coeff->data, a->input->data + (size_t)n * in, y, out, 1, in, 0);
        if (a->use_biases == 1)
            for (int i = 0; i < out; i++) y[i] = y[i] + a->bias->data[i];
    }
}

void NAME(orc_linear_wg)(const LIN_ARGS *a, int ns) {
    int in = a->input->dim, out = a->output->dim;
    size_t wn = (size_t)in * out;
    T *one = (T *)malloc(wn * sizeof(T));
    float *sum = (float *)calloc(wn, sizeof(float));
    float *bsum = (float *)calloc((size_t)out, sizeof(float));
    for (int n = 0; n < ns; n++) {
        const T *dy = a->output->diff + (size_t)n * out;
        NAME(mm_core)(dy, a->input->data + (size_t)n * in, one, out, in, 1, 0);
        for (size_t i = 0; i < wn; i++) sum[i] += (float)one[i];
        for (int i = 0; i < out; i++) bsum[i] += (float)dy[i];
    }
    for (size_t i = 0; i < wn; i++) a->coeff->diff[i] = (T)sum[i];
    if (a->use_biases == 1)
        for (int i = 0; i < out; i++) a->bias->diff[i] = (T)bsum[i];
    free(one); free(sum); free(bsum);
}

void NAME(orc_linear_ig)(const LIN_ARGS *a, int ns) {
    int in = a->input->dim, out = a->output->dim;
    for (int n = 0; n < ns; n++)
        NAME(mm_core)(a->output->diff + (size_t)n * out, a->coeff->data, a->input->diff + (size_t)n * in, 1, in, out,
                      0);
}

/* ---- transposition and layout: lib/sources/pulp_train_utils_fp32.c:39-76
 * (transpose_matrix: out[j*N+i] = in[i*M+j]), :79-183 (n-d transpose, output
 * axis i = input axis transposed_axes[i]), :821-927 (layout change = transpose
 * into the buffer, copy back), :929-984 (pad_tensor).  pad_tensor's border
 * test in the reference (wt > W, ht > H, :957) holds only for pads of 1; the
 * true bound is used. */
void NAME(orc_transpose_matrix)(void *p) {
    TR_ARGS *a = (TR_ARGS *)p;
    for (int i = 0; i < a->N; i++)
        for (int j = 0; j < a->M; j++) a->out_matrix[(size_t)j * a->N + i] = a->in_matrix[(size_t)i * a->M + j];
}

void NAME(orc_transpose)(void *p) {
    TR_ARGS *a = (TR_ARGS *)p;
    int nd = a->n_dim;
    int tr_indexes[16], prod[16];
    size_t n_elements = 1;
    for (int i = 0; i < nd; i++) n_elements *= (size_t)a->dim[i];
    for (int i = 0; i < nd; i++) tr_indexes[a->transposed_axes[i]] = i;
    prod[nd - 1] = 1;
    for (int i = nd - 2; i >= 0; i--) prod[i] = prod[i + 1] * a->dim[a->transposed_axes[i + 1]];
    for (size_t i = 0; i < n_elements; i++) {
        size_t idx = i, new_index = 0;
        for (int j = nd - 1; j >= 0; j--) {
            new_index += (idx % a->dim[j]) * (size_t)prod[tr_indexes[j]];
            idx /= a->dim[j];
        }
        a->out_matrix[new_index] = a->in_matrix[i];
    }
}

static void NAME(relayout_one)(T *t, T *buf, int rows, int cols) {
    for (int i = 0; i < rows; i++)
        for (int j = 0; j < cols; j++) buf[(size_t)j * rows + i] = t[(size_t)i * cols + j];
    memcpy(t, buf, (size_t)rows * cols * sizeof(T));
}

void NAME(orc_CHW_to_HWC)(void *p) {
    LAY_ARGS *a = (LAY_ARGS *)p;
    int C = (uint16_t)a->tensor->C, H = (uint16_t)a->tensor->H, W = (uint16_t)a->tensor->W;
    if ((uint8_t)a->transpose_data == 1) NAME(relayout_one)(a->tensor->data, a->transp_buffer, C, H * W);
    if ((uint8_t)a->transpose_grad == 1) NAME(relayout_one)(a->tensor->diff, a->transp_buffer, C, H * W);
}

void NAME(orc_HWC_to_CHW)(void *p) {
    LAY_ARGS *a = (LAY_ARGS *)p;
    int C = (uint16_t)a->tensor->C, H = (uint16_t)a->tensor->H, W = (uint16_t)a->tensor->W;
    if ((uint8_t)a->transpose_data == 1) NAME(relayout_one)(a->tensor->data, a->transp_buffer, H * W, C);
    if ((uint8_t)a->transpose_grad == 1) NAME(relayout_one)(a->tensor->diff, a->transp_buffer, H * W, C);
}

void NAME(orc_pad_tensor)(void *p) {
    PAD_ARGS *a = (PAD_ARGS *)p;
    int C = a->C, H = a->H, W = a->W, L = a->T_LPAD, U = a->T_UPAD;
    int Ho = H + a->T_UPAD + a->T_DPAD, Wo = W + a->T_LPAD + a->T_RPAD;
    for (int ch = 0; ch < C; ch++)
        for (int ht = 0; ht < Ho; ht++)
            for (int wt = 0; wt < Wo; wt++) {
                int h = ht - U, w = wt - L;
                int inside = h >= 0 && h < H && w >= 0 && w < W;
                if (a->HWC_lay == 0)
                    a->dest[wt + ht * Wo + (size_t)ch * Ho * Wo] = inside ? a->source[w + h * W + (size_t)ch * H * W] : (T)0;
                else
                    a->dest[ch + (size_t)wt * C + (size_t)ht * C * Wo] =
                        inside ? a->source[ch + (size_t)w * C + (size_t)h * C * W] : (T)0;
            }
}

/* ---- streaming helpers: lib/sources/pulp_train_utils_fp32.c:186-219 */
void NAME(orc_vect_sum)(const T *x, const T *y, T *z, int n) {
    for (int i = 0; i < n; i++) z[i] = x[i] + y[i];
}

#undef IDX_ACT
#undef IDX_WGT
