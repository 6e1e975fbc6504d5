/*
 * TEST INFRASTRUCTURE - CPU oracle of the fp32 multi-head self-attention step.
 *
 * Restates the operation list of lib/sources/pulp_mhsa_fp32.c (forward :20-646,
 * backward :648-1747) with the helpers it calls: `mm` (k-sequential fp32 sums,
 * lib/sources/pulp_matmul_fp32.c:190), mm_bias_add_transposed with the per-row
 * branch (lib/sources/pulp_train_utils_fp32.c:1286; the reference leaves the
 * selector `t` unset, the golden model tests/test_mhsa_fp32/utils/mhsa.py adds
 * the bias per feature = per row), pulp_scalar_mul_fp32_cl (:1263), the softmax
 * forward/backward of lib/sources/pulp_act_fp32.c:187,335 over
 * pulp_row_max/exp_sum/row_div/sm_bw_op_1/2 (lib/sources/pulp_train_utils_fp32.c:1046-1189),
 * fastexp_gist (:1223) and q_rsqrt (:1234, restated with a 32-bit integer: the
 * reference's `long` is 8 bytes on x86-64).  The reference transposes
 * matrices into a scratch buffer before most products; transposition moves
 * values without changing them, so the products below index the operands in
 * place and keep only the summation order of `mm`.
 *
 * Only tests, the smoke check and the benchmark's CPU-baseline leg load this.
 *
 * Pinning (tests/test_oracle_mhsa.py): forward against a float64 torch model
 * of tests/test_mhsa_fp32/utils/mhsa.py with the approximate exponential
 * evaluated in float32 from its definition; backward against torch autograd
 * through that model with the exact softmax Jacobian taken at the oracle's
 * own softmax output; fastexp against exp() within its published error and
 * bit-exactly against an integer evaluation; q_rsqrt against 1/sqrt.
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#include "ptl_structs.h"

#define GIST_A 12102203.17133801f /* lib/include/pulp_train_defines.h:85-88 */
#define GIST_B 1064986823.010288f
#define GIST_C 8388608
#define GIST_D 2139095040

float orc_fastexp_gist(float x) {
    x = GIST_A * x + GIST_B;
    if (x < GIST_C || x > GIST_D) x = (x < GIST_C) ? 0.0f : GIST_D;
    uint32_t n = (uint32_t)(x);
    float r;
    memcpy(&r, &n, 4);
    return r;
}

float orc_q_rsqrt(float number) {
    int32_t i;
    float x2 = number * 0.5f, y = number;
    memcpy(&i, &y, 4);
    i = 0x5f3759df - (i >> 1);
    memcpy(&y, &i, 4);
    y = y * (1.5f - (x2 * y * y));
    return y;
}

/* C[i][j] = sum_k A(i,k) * B(k,j), k ascending in one fp32 accumulator; operands addressed by strides. */
static void mm_strided(const float *A, long a_i, long a_k, const float *B, long b_k, long b_j, float *C, long c_i,
                       long c_j, int N, int M, int K) {
#pragma omp parallel for schedule(static)
    for (int i = 0; i < N; ++i)
        for (int j = 0; j < M; ++j) {
            float t = 0.f;
            for (int k = 0; k < K; ++k) t += A[i * a_i + k * a_k] * B[k * b_k + j * b_j];
            C[i * c_i + j * c_j] = t;
        }
}

/* out = softmax over each row of in (H rows of W), approximate exponential. */
void orc_softmax_fw_fp32(void *p) {
    struct softmax_args *a = (struct softmax_args *)p;
    const int H = a->H, W = a->W;
    for (int i = 0; i < H; ++i) {
        float mx = -340282346638528859811704183484516925440.0f, s = 0.f;
        for (int j = 0; j < W; ++j)
            if (mx < a->input_data[i * W + j]) mx = a->input_data[i * W + j];
        for (int j = 0; j < W; ++j) {
            float o = orc_fastexp_gist(a->input_data[i * W + j] - mx);
            a->output_data[i * W + j] = o;
            s += o;
        }
        for (int j = 0; j < W; ++j) a->output_data[i * W + j] = a->output_data[i * W + j] / s;
        if (a->maxes) a->maxes[i] = mx;
        if (a->sums) a->sums[i] = s;
    }
}

/* in_diff = (out_diff - sum_j out_diff*out) * out, row by row. */
void orc_softmax_bw_fp32(void *p) {
    struct softmax_args *a = (struct softmax_args *)p;
    const int H = a->H, W = a->W;
    for (int i = 0; i < H; ++i) {
        float s = 0.f;
        for (int j = 0; j < W; ++j) s += a->output_diff[i * W + j] * a->output_data[i * W + j];
        for (int j = 0; j < W; ++j)
            a->input_diff[i * W + j] = (a->output_diff[i * W + j] - s) * a->output_data[i * W + j];
        if (a->sums) a->sums[i] = s;
    }
}

static void dims(const struct Mhsa_args *a, int *L, int *E, int *F, int *H) {
    *L = a->input->H;
    *E = a->input->W;
    *F = a->attention_map->W;
    *H = *F / a->n_heads;
}

void orc_mhsa_fw_fp32(const struct Mhsa_args *a, int ns) {
    int L, E, F, H;
    dims(a, &L, &E, &F, &H);
    const int heads = a->n_heads;
    const float scaling = orc_q_rsqrt((float)H);
    float *tmp = (float *)malloc(sizeof(float) * (size_t)L * L);
    for (int b = 0; b < ns; ++b) {
        const float *X = a->input->data + (size_t)b * E * L;
        float *Q = a->q->data + (size_t)b * F * L, *Kk = a->k->data + (size_t)b * F * L;
        float *V = a->v->data + (size_t)b * F * L, *att = a->attention_map->data + (size_t)b * F * L;
        float *P = a->softmax_buffer->data + (size_t)b * heads * L * L;
        float *Y = a->output->data + (size_t)b * E * L;
        const struct blob *wq[3] = {a->coeff_in_q, a->coeff_in_k, a->coeff_in_v};
        const struct blob *bq[3] = {a->bias_in_q, a->bias_in_k, a->bias_in_v};
        float *dst[3] = {Q, Kk, V};
        for (int j = 0; j < 3; ++j) {
            /* T0 + M1: dst[F x L] = (W^T)[F x E] . X[E x L]; W stored E x F (:86-127) */
            mm_strided(wq[j]->data, 1, F, X, L, 1, dst[j], L, 1, F, L, E);
            if (bq[j] && bq[j]->data)
                for (int f = 0; f < F; ++f)
                    for (int l = 0; l < L; ++l) dst[j][f * L + l] = dst[j][f * L + l] + bq[j]->data[f];
        }
        for (int h = 0; h < heads; ++h) {
            const float *q = Q + (size_t)h * H * L, *k = Kk + (size_t)h * H * L, *v = V + (size_t)h * H * L;
            float *Ph = P + (size_t)h * L * L;
            /* T1 + M2: S[key][query] = sum_d k[d][key] q[d][query] (:349-376); scaled (:424-431);
             * T2: row = query, column = key (:447-456) */
            mm_strided(k, 1, L, q, L, 1, tmp, 1, L, L, L, H); /* written transposed: tmp[query][key] */
            for (int i = 0; i < L * L; ++i) tmp[i] = tmp[i] * scaling;
            struct softmax_args sm = {0};
            sm.input_data = tmp;
            sm.output_data = Ph;
            sm.H = L;
            sm.W = L;
            orc_softmax_fw_fp32(&sm);
            /* T3 + M3: att[d][query] = sum_key v[d][key] P[query][key] (:520-556) */
            mm_strided(v, L, 1, Ph, 1, L, att + (size_t)h * H * L, L, 1, H, L, L);
        }
        /* M4: Y[E x L] = Wout[E x F] . att[F x L] (:599-609) */
        mm_strided(a->coeff_out->data, F, 1, att, L, 1, Y, L, 1, E, L, F);
    }
    free(tmp);
}

void orc_mhsa_bw_fp32(const struct Mhsa_args *a, int ns) {
    int L, E, F, H;
    dims(a, &L, &E, &F, &H);
    const int heads = a->n_heads;
    const float scaling = orc_q_rsqrt((float)H);
    float *grad = (float *)malloc(sizeof(float) * (size_t)L * L);
    float *tmp = (float *)malloc(sizeof(float) * (size_t)(E > F ? E : F) * (L > E ? L : E));
    float *acc = (float *)malloc(sizeof(float) * (size_t)E * F);
    float *dWo = a->coeff_out->diff;
    float *dW[3] = {a->coeff_in_q->diff, a->coeff_in_k->diff, a->coeff_in_v->diff};
    const float *Wd[3] = {a->coeff_in_q->data, a->coeff_in_k->data, a->coeff_in_v->data};
    for (int b = 0; b < ns; ++b) {
        const float *X = a->input->data + (size_t)b * E * L;
        const float *dY = a->output->diff + (size_t)b * E * L;
        float *dX = a->input->diff + (size_t)b * E * L;
        const float *att = a->attention_map->data + (size_t)b * F * L;
        float *datt = a->attention_map->diff + (size_t)b * F * L;
        const float *P = a->softmax_buffer->data + (size_t)b * heads * L * L;
        float *dP = a->softmax_buffer->diff + (size_t)b * heads * L * L;
        const float *QKV[3] = {a->q->data + (size_t)b * F * L, a->k->data + (size_t)b * F * L,
                               a->v->data + (size_t)b * F * L};
        float *dQKV[3] = {a->q->diff + (size_t)b * F * L, a->k->diff + (size_t)b * F * L,
                          a->v->diff + (size_t)b * F * L};
        /* T1 + M1: dWout[E x F] = dY[E x L] . att^T (:742-760); summed over the samples of a batch */
        mm_strided(dY, L, 1, att, 1, L, b == 0 ? dWo : acc, F, 1, E, F, L);
        if (b)
            for (int i = 0; i < E * F; ++i) dWo[i] += acc[i];
        /* T2 + M2: datt[F x L] = Wout^T . dY (:816-834) */
        mm_strided(a->coeff_out->data, 1, F, dY, L, 1, datt, L, 1, F, L, E);
        for (int h = 0; h < heads; ++h) {
            const float *q = QKV[0] + (size_t)h * H * L, *k = QKV[1] + (size_t)h * H * L;
            const float *v = QKV[2] + (size_t)h * H * L;
            const float *Ph = P + (size_t)h * L * L;
            float *dPh = dP + (size_t)h * L * L;
            const float *da = datt + (size_t)h * H * L;
            /* M3: dv[d][key] = sum_query da[d][query] P[query][key] (:884-902) */
            mm_strided(da, L, 1, Ph, L, 1, dQKV[2] + (size_t)h * H * L, L, 1, H, L, L);
            /* T3 + M4 + T4/C1: dP[query][key] = sum_d v[d][key] da[d][query] (:958-1060) */
            mm_strided(v, 1, L, da, L, 1, dPh, 1, L, L, L, H);
            /* SM (:1071-1080), T5/C2 keep the (query, key) orientation of this restatement; scaling (:1176-1183) */
            struct softmax_args sm = {0};
            sm.input_diff = grad;
            sm.output_data = (float *)Ph;
            sm.output_diff = dPh;
            sm.H = L;
            sm.W = L;
            orc_softmax_bw_fp32(&sm);
            for (int i = 0; i < L * L; ++i) grad[i] = grad[i] * scaling;
            /* T6 + M5 + T7/C3: dk[d][key] = sum_query grad[query][key] q[d][query] (:1244-1330) */
            mm_strided(grad, 1, L, q, 1, L, tmp, 1, L, L, H, L); /* tmp[d][key] */
            memcpy(dQKV[1] + (size_t)h * H * L, tmp, sizeof(float) * (size_t)H * L);
            /* M6: dq[d][query] = sum_key k[d][key] grad[query][key] (:1342-1360) */
            mm_strided(k, L, 1, grad, 1, L, dQKV[0] + (size_t)h * H * L, L, 1, H, L, L);
        }
        for (int j = 0; j < 3; ++j) {
            /* T8 + M7: dW[F x E] = d{q,k,v}[F x L] . X^T (:1425-1560) */
            mm_strided(dQKV[j], L, 1, X, 1, L, b == 0 ? dW[j] : acc, E, 1, F, E, L);
            if (b)
                for (int i = 0; i < E * F; ++i) dW[j][i] += acc[i];
            /* M8 + SUM: dX[E x L] += W[E x F] . d{q,k,v}[F x L] (:1589-1745) */
            mm_strided(Wd[j], F, 1, dQKV[j], L, 1, tmp, L, 1, E, L, F);
            for (int i = 0; i < E * L; ++i) dX[i] = dX[i] + tmp[i];
        }
    }
    free(grad);
    free(tmp);
    free(acc);
}
