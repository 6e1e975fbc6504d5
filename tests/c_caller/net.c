/*
 * A C caller in the style of the reference's per-test net.c
 * (tests/test_conv2d_fp32/net.c:423-450, tests/test_linear_fp32/net.c,
 * tests/test_conv_pw_dw_fp32/net.c): static tensors, blobs and an argument
 * struct filled in by hand, the layer's forward and backward entry points
 * called by name.  It is compiled by the tests against include/ptl_api.h and
 * linked with libptl_hip.so; nothing else of the library is visible to it.
 *
 * usage: net <conv2d|linear|pw|dw> <out-file>
 * The inputs (seeded, uniform in [-1, 1)) and the results are written to
 * <out-file> as raw arrays in the order x, w, dy, y, dw, dx; the exit code is
 * 0 on success, 3 when the library reports that a call failed.
 */
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "ptl_api.h"

#define PI_L1 /* the reference places its tensors in cluster memory with this attribute */

/* BASELINE config 1: Conv2D 16 -> 32 channels, 32x32, 3x3, stride 1, pad 1, fp32 */
#define C_CI 16
#define C_CO 32
#define C_H 32
#define C_K 3
PI_L1 static float c_in[C_CI * C_H * C_H], c_in_diff[C_CI * C_H * C_H];
PI_L1 static float c_w[C_CO * C_CI * C_K * C_K], c_w_diff[C_CO * C_CI * C_K * C_K];
PI_L1 static float c_out[C_CO * C_H * C_H], c_out_diff[C_CO * C_H * C_H];

/* Linear 256 -> 128, fp32 */
#define L_IN 256
#define L_OUT 128
PI_L1 static float l_in[L_IN], l_in_diff[L_IN], l_w[L_OUT * L_IN], l_w_diff[L_OUT * L_IN], l_out[L_OUT],
    l_out_diff[L_OUT];

/* Pointwise 16 -> 24 on 10x10 and depthwise 3x3 on 8 x 12 x 12, fp32 */
#define P_CI 16
#define P_CO 24
#define P_HW 100
PI_L1 static float p_in[P_CI * P_HW], p_in_diff[P_CI * P_HW], p_w[P_CO * P_CI], p_w_diff[P_CO * P_CI],
    p_out[P_CO * P_HW], p_out_diff[P_CO * P_HW];
#define D_C 8
#define D_H 12
#define D_HO 10
PI_L1 static float d_in[D_C * D_H * D_H], d_in_diff[D_C * D_H * D_H], d_w[D_C * 9], d_w_diff[D_C * 9],
    d_out[D_C * D_HO * D_HO], d_out_diff[D_C * D_HO * D_HO];

static unsigned long long rng_state = 0xC0DE0001ull;

static float next_uniform(void) { /* SplitMix64 -> [-1, 1) */
    unsigned long long z = (rng_state += 0x9E3779B97F4A7C15ull);
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    z ^= z >> 31;
    return (float)(-1.0 + 2.0 * (double)(z >> 11) * (1.0 / 9007199254740992.0));
}

static void fill(float *p, int n) {
    for (int i = 0; i < n; i++) p[i] = next_uniform();
}

static int dump(FILE *f, const float *p, int n) { return fwrite(p, sizeof(float), (size_t)n, f) == (size_t)n ? 0 : 1; }

static int check(const char *what) {
    if (ptl_last_status() == 0) return 0;
    fprintf(stderr, "%s failed: %s\n", what, ptl_last_error());
    return 3;
}

static int run_conv2d(FILE *f) {
    struct blob b_in = {c_in, c_in_diff, C_CI * C_H * C_H, C_H, C_H, C_CI}; /* data, diff, dim, W, H, C */
    struct blob b_w = {c_w, c_w_diff, C_CO * C_CI * C_K * C_K, C_K, C_K, C_CI};
    struct blob b_out = {c_out, c_out_diff, C_CO * C_H * C_H, C_H, C_H, C_CO};
    struct Conv2D_args a;
    memset(&a, 0, sizeof a);
    a.input = &b_in; a.coeff = &b_w; a.bias = NULL; a.output = &b_out;
    a.Lpad = a.Rpad = a.Upad = a.Dpad = 1;
    a.stride_h = a.stride_w = 1;
    a.i2c_buffer = NULL; a.bt_buffer = NULL; /* im2col is implicit: no buffers needed */
    a.HWC = 0; a.USE_BIASES = 0; a.USE_IM2COL = 1; a.USE_DMA_IM2COL = 0;
    fill(c_in, C_CI * C_H * C_H); fill(c_w, C_CO * C_CI * C_K * C_K); fill(c_out_diff, C_CO * C_H * C_H);
    pulp_conv2d_fp32_fw_cl(&a);
    if (check("pulp_conv2d_fp32_fw_cl")) return 3;
    pulp_conv2d_fp32_bw_cl(&a); /* weight + input gradient, honours skip_* */
    if (check("pulp_conv2d_fp32_bw_cl")) return 3;
    return dump(f, c_in, C_CI * C_H * C_H) | dump(f, c_w, C_CO * C_CI * C_K * C_K) | dump(f, c_out_diff, C_CO * C_H * C_H) |
           dump(f, c_out, C_CO * C_H * C_H) | dump(f, c_w_diff, C_CO * C_CI * C_K * C_K) | dump(f, c_in_diff, C_CI * C_H * C_H);
}

static int run_linear(FILE *f) {
    struct blob b_in = {l_in, l_in_diff, L_IN, L_IN, 1, 1};
    struct blob b_w = {l_w, l_w_diff, L_IN * L_OUT, L_IN, L_OUT, 1};
    struct blob b_out = {l_out, l_out_diff, L_OUT, L_OUT, 1, 1};
    struct Linear_args a;
    memset(&a, 0, sizeof a);
    a.input = &b_in; a.coeff = &b_w; a.bias = NULL; a.output = &b_out; a.use_biases = 0;
    fill(l_in, L_IN); fill(l_w, L_IN * L_OUT); fill(l_out_diff, L_OUT);
    pulp_linear_fp32_fw_cl(&a);
    if (check("pulp_linear_fp32_fw_cl")) return 3;
    pulp_linear_fp32_bw_param_grads_cl(&a);
    if (check("pulp_linear_fp32_bw_param_grads_cl")) return 3;
    pulp_linear_fp32_bw_input_grads_cl(&a);
    if (check("pulp_linear_fp32_bw_input_grads_cl")) return 3;
    return dump(f, l_in, L_IN) | dump(f, l_w, L_IN * L_OUT) | dump(f, l_out_diff, L_OUT) | dump(f, l_out, L_OUT) |
           dump(f, l_w_diff, L_IN * L_OUT) | dump(f, l_in_diff, L_IN);
}

static int run_pw(FILE *f) {
    struct blob b_in = {p_in, p_in_diff, P_CI * P_HW, 10, 10, P_CI};
    struct blob b_w = {p_w, p_w_diff, P_CO * P_CI, 1, 1, P_CI};
    struct blob b_out = {p_out, p_out_diff, P_CO * P_HW, 10, 10, P_CO};
    struct PointWise_Conv_args a;
    memset(&a, 0, sizeof a);
    a.input = &b_in; a.coeff = &b_w; a.output = &b_out; a.transpose_buffer = NULL; a.HWC = 0;
    fill(p_in, P_CI * P_HW); fill(p_w, P_CO * P_CI); fill(p_out_diff, P_CO * P_HW);
    pulp_conv_pw_fp32_fw_cl(&a);
    if (check("pulp_conv_pw_fp32_fw_cl")) return 3;
    pulp_conv_pw_fp32_bw_cl(&a);
    if (check("pulp_conv_pw_fp32_bw_cl")) return 3;
    return dump(f, p_in, P_CI * P_HW) | dump(f, p_w, P_CO * P_CI) | dump(f, p_out_diff, P_CO * P_HW) |
           dump(f, p_out, P_CO * P_HW) | dump(f, p_w_diff, P_CO * P_CI) | dump(f, p_in_diff, P_CI * P_HW);
}

static int run_dw(FILE *f) {
    struct blob b_in = {d_in, d_in_diff, D_C * D_H * D_H, D_H, D_H, D_C};
    struct blob b_w = {d_w, d_w_diff, D_C * 9, 3, 3, 1};
    struct blob b_out = {d_out, d_out_diff, D_C * D_HO * D_HO, D_HO, D_HO, D_C};
    struct DepthWise_Conv_args a;
    memset(&a, 0, sizeof a);
    a.input = &b_in; a.coeff = &b_w; a.output = &b_out;
    a.stride_h = a.stride_w = 1;
    fill(d_in, D_C * D_H * D_H); fill(d_w, D_C * 9); fill(d_out_diff, D_C * D_HO * D_HO);
    pulp_conv_dw_fp32_fw_cl(&a);
    if (check("pulp_conv_dw_fp32_fw_cl")) return 3;
    pulp_conv_dw_fp32_bw_cl(&a);
    if (check("pulp_conv_dw_fp32_bw_cl")) return 3;
    return dump(f, d_in, D_C * D_H * D_H) | dump(f, d_w, D_C * 9) | dump(f, d_out_diff, D_C * D_HO * D_HO) |
           dump(f, d_out, D_C * D_HO * D_HO) | dump(f, d_w_diff, D_C * 9) | dump(f, d_in_diff, D_C * D_H * D_H);
}

int main(int argc, char **argv) {
    FILE *f;
    int rc = 2;
    if (argc != 3) {
        fprintf(stderr, "usage: %s <conv2d|linear|pw|dw> <out-file>\n", argv[0]);
        return 2;
    }
    f = fopen(argv[2], "wb");
    if (!f) return 2;
    if (!strcmp(argv[1], "conv2d")) rc = run_conv2d(f);
    else if (!strcmp(argv[1], "linear")) rc = run_linear(f);
    else if (!strcmp(argv[1], "pw")) rc = run_pw(f);
    else if (!strcmp(argv[1], "dw")) rc = run_dw(f);
    fclose(f);
    if (rc == 0) printf("%s ok\n", argv[1]);
    return rc;
}
