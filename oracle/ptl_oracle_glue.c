/*
 * TEST INFRASTRUCTURE - CPU oracle of the layers around the matmul core in a ResNet-style step.
 *
 * Restates, loop for loop: ReLU (lib/sources/pulp_act_fp32.c:95-129), the residual connection
 * (lib/sources/pulp_residual_fp32.c:26-113), average pooling (lib/sources/pulp_pooling_fp32.c:24-122),
 * cross-entropy over raw logits (lib/sources/pulp_losses_fp32.c:26-138), gradient descent
 * (lib/sources/pulp_optimizers_fp32.c:26-104), batch normalisation forward
 * (lib/sources/pulp_batchnorm_fp32.c:34-114), and their fp16 twins with the reference's arithmetic types
 * (fp16 accumulator in pooling and in the optimizer, float inside the loss: pulp_pooling_fp16.c:24-122,
 * pulp_optimizers_fp16.c:26, pulp_losses_fp16.c:26-136).  Batched forms loop over the samples.
 *
 * Only tests, the smoke check and the benchmark's CPU-baseline leg load this.
 *
 * Pinning (tests/test_oracle_glue.py): torch relu / avg_pool2d / cross_entropy (soft targets) /
 * batch_norm and their autograd in float64, a hand-written SGD update in numpy float64.
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

#include "ptl_structs.h"

#define GLUE(T, SFX, BLOB, ACT, SKIP, POOL, LOSS, OPT)                                                        \
    void orc_relu_##SFX(const ACT *a, int ns, int step) {                                                     \
        const long n = (long)ns * a->input->dim;                                                              \
        const T *x = a->input->data;                                                                          \
        if (step == 0) {                                                                                      \
            T *y = a->output->data;                                                                           \
            for (long i = 0; i < n; ++i) y[i] = x[i] > 0 ? x[i] : (T)0;                                       \
        } else {                                                                                              \
            const T *dy = a->output->diff;                                                                    \
            T *dx = a->input->diff;                                                                           \
            for (long i = 0; i < n; ++i) dx[i] = x[i] > 0 ? dy[i] : (T)0;                                     \
        }                                                                                                     \
    }                                                                                                         \
    void orc_residual_##SFX(const SKIP *a, int ns, int step) {                                                \
        const long n = (long)ns * a->output->dim;                                                             \
        if (step == 0) {                                                                                      \
            for (long i = 0; i < n; ++i) a->output->data[i] = a->skip->data[i] + a->lout->data[i];            \
        } else if (step == 1) {                                                                               \
            if (a->skip_in_grad == 0)                                                                         \
                for (long i = 0; i < n; ++i) a->skip->diff[i] = a->output->diff[i] + a->skip->diff[i];        \
        } else {                                                                                              \
            for (long i = 0; i < n; ++i) a->lout->diff[i] = a->output->diff[i];                               \
        }                                                                                                     \
    }                                                                                                         \
    void orc_avgpool_##SFX(const POOL *a, int ns, int step) {                                                 \
        const int W = a->input->W, H = a->input->H, C = a->input->C, Ho = a->output->H, Wo = a->output->W;    \
        const int Hk = a->Hker, Wk = a->Wker, Hs = a->Hstride, Ws = a->Wstride;                               \
        const int Hact = (H - Hk + Hs) / Hs, Wact = (W - Wk + Ws) / Ws, HW = H * W, HWk = Hk * Wk,            \
                  HWo = Ho * Wo;                                                                              \
        for (long k = 0; k < (long)ns * C; ++k) {                                                             \
            if (step == 0) {                                                                                  \
                for (int ha = 0; ha < Hact; ++ha)                                                             \
                    for (int wa = 0; wa < Wact; ++wa) {                                                       \
                        T s = 0;                                                                              \
                        for (int hk = 0; hk < Hk; ++hk)                                                       \
                            for (int wk = 0; wk < Wk; ++wk)                                                   \
                                s += a->input->data[wk + wa * Ws + (hk + ha * Hs) * W + k * HW];              \
                        a->output->data[wa + ha * Wo + k * HWo] = s / HWk;                                    \
                    }                                                                                         \
            } else {                                                                                          \
                for (int hw = 0; hw < HW; ++hw) a->input->diff[k * HW + hw] = 0;                              \
                for (int ho = 0; ho < Ho; ++ho)                                                               \
                    for (int wo = 0; wo < Wo; ++wo)                                                           \
                        for (int hk = 0; hk < Hk; ++hk)                                                       \
                            for (int wk = 0; wk < Wk; ++wk)                                                   \
                                a->input->diff[(wk + wo * Ws) + (hk + ho * Hs) * W + k * HW] +=               \
                                    a->output->diff[wo + ho * Wo + k * HWo] / HWk;                            \
            }                                                                                                 \
        }                                                                                                     \
    }                                                                                                         \
    void orc_cross_entropy_##SFX(const LOSS *a, int ns, int step) {                                           \
        const int n = a->output->dim;                                                                         \
        for (int b = 0; b < ns; ++b) {                                                                        \
            const T *z = a->output->data + (long)b * n, *y = a->target + (long)b * n;                         \
            float mx = (float)z[0];                                                                           \
            for (int i = 1; i < n; ++i)                                                                       \
                if ((float)z[i] > mx) mx = (float)z[i];                                                       \
            float se = 0.0f;                                                                                  \
            for (int i = 0; i < n; ++i) se += expf((float)z[i] - mx);                                         \
            float sy = 0.0f, dot = 0.0f;                                                                      \
            for (int i = 0; i < n; ++i) {                                                                     \
                dot += (float)y[i] * (float)z[i];                                                             \
                sy += (float)y[i];                                                                            \
            }                                                                                                 \
            if (step == 0) {                                                                                  \
                if (sizeof(T) == 4 && sy == 0.0f) sy = 1.0f;                                                  \
                a->wr_loss[b] = (T)(-(dot - (logf(se) + mx) * sy));                                           \
            } else {                                                                                          \
                if (sy == 0.0f) sy = 1.0f;                                                                    \
                const float inv = 1.0f / se;                                                                  \
                T *g = a->output->diff + (long)b * n;                                                         \
                for (int i = 0; i < n; ++i) g[i] = (T)((expf((float)z[i] - mx) * inv) * sy - (float)y[i]);    \
            }                                                                                                 \
        }                                                                                                     \
    }                                                                                                         \
    void orc_gradient_descent_##SFX(const OPT *a) {                                                           \
        const T lr = a->learning_rate, lambda = a->weight_decay_lambda;                                       \
        for (int part = 0; part < 2; ++part) {                                                                \
            if (part == 1 && a->use_biases != 1) break;                                                       \
            const BLOB *bl = part ? a->biases : a->weights;                                                   \
            T *w = bl->data, *g = bl->diff;                                                                   \
            for (int i = 0; i < bl->dim; ++i) {                                                               \
                if (lambda != 0) g[i] += lambda * w[i];                                                       \
                w[i] -= lr * g[i];                                                                            \
            }                                                                                                 \
        }                                                                                                     \
    }

GLUE(float, fp32, struct blob, struct act_args, struct SkipConn_args, struct pool_args, struct loss_args,
     struct optim_args)
GLUE(_Float16, fp16, struct blob_fp16, struct act_args_fp16, struct SkipConn_args_fp16, struct pool_args_fp16,
     struct loss_args_fp16, struct optim_args_fp16)

/* Batch normalisation.  Forward: lib/sources/pulp_batchnorm_fp32.c:34-114 (sums of x and x^2 per channel over
 * B x H x W, deviation = sqrt((s2 - 2 s1 mean) / n + mean^2 + eps)).  The reference has no backward pass and no
 * fp16 variant; those restate the textbook gradient of that forward,
 *   xh = (x - mean) / sd, dbeta = sum dy, dgamma = sum dy xh, dx = gamma / sd (dy - dbeta / n - xh dgamma / n),
 * with fp32 sums: parity unpinned against the reference (it has nothing to compare with), pinned against torch
 * autograd in float64 by tests/test_oracle_glue.py. */
#define BATCH_NORM(T, SFX, ARGS)                                                                          \
    static void bn_stats_##SFX(const ARGS *a, int c, float *mean, float *sd) {                            \
        const T *in = a->input->data;                                                                     \
        const int B = a->B, C = a->C, HW = a->H * a->W, n = B * HW;                                        \
        float s1 = 0.0f, s2 = 0.0f;                                                                       \
        for (int b = 0; b < B; ++b)                                                                       \
            for (int hw = 0; hw < HW; ++hw) {                                                             \
                const float v = (float)in[b * C * HW + c * HW + hw];                                      \
                s1 += v;                                                                                  \
                s2 += v * v;                                                                              \
            }                                                                                             \
        *mean = s1 / n;                                                                                   \
        *sd = sqrtf(((s2 - 2 * s1 * *mean) / n) + (*mean * *mean) + (float)a->eps[0]);                    \
    }                                                                                                     \
    void orc_batch_norm_fw_##SFX(const ARGS *a) {                                                         \
        const T *in = a->input->data;                                                                     \
        T *out = a->output->data;                                                                         \
        const int B = a->B, C = a->C, HW = a->H * a->W;                                                    \
        for (int c = 0; c < C; ++c) {                                                                     \
            float mean, sd;                                                                               \
            bn_stats_##SFX(a, c, &mean, &sd);                                                             \
            for (int b = 0; b < B; ++b)                                                                   \
                for (int hw = 0; hw < HW; ++hw) {                                                         \
                    const int idx = b * C * HW + c * HW + hw;                                             \
                    out[idx] = (T)((((float)in[idx] - mean) / sd) * (float)a->weight_data[c] +            \
                                   (float)a->bias_data[c]);                                               \
                }                                                                                         \
        }                                                                                                 \
    }                                                                                                     \
    void orc_batch_norm_bw_##SFX(const ARGS *a) {                                                         \
        const T *in = a->input->data, *dy = a->output->diff;                                              \
        const int B = a->B, C = a->C, HW = a->H * a->W, n = B * HW;                                        \
        for (int c = 0; c < C; ++c) {                                                                     \
            float mean, sd, db = 0.0f, dg = 0.0f;                                                         \
            bn_stats_##SFX(a, c, &mean, &sd);                                                             \
            for (int b = 0; b < B; ++b)                                                                   \
                for (int hw = 0; hw < HW; ++hw) {                                                         \
                    const int idx = b * C * HW + c * HW + hw;                                             \
                    db += (float)dy[idx];                                                                 \
                    dg += (float)dy[idx] * (((float)in[idx] - mean) / sd);                                \
                }                                                                                         \
            if (!a->skip_wg_grad) {                                                                       \
                if (a->coeff) a->coeff->diff[c] = (T)dg;                                                  \
                if (a->bias) a->bias->diff[c] = (T)db;                                                    \
            }                                                                                             \
            if (a->skip_in_grad) continue;                                                                \
            for (int b = 0; b < B; ++b)                                                                   \
                for (int hw = 0; hw < HW; ++hw) {                                                         \
                    const int idx = b * C * HW + c * HW + hw;                                             \
                    const float xh = ((float)in[idx] - mean) / sd;                                        \
                    a->input->diff[idx] =                                                                 \
                        (T)(((float)a->weight_data[c] / sd) * ((float)dy[idx] - db / n - xh * dg / n));   \
                }                                                                                         \
        }                                                                                                 \
    }

BATCH_NORM(float, fp32, struct BatchNorm_args_fp32)
BATCH_NORM(_Float16, fp16, struct BatchNorm_args_fp16)
