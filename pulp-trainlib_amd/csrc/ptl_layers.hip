// Conv2D, pointwise convolution and Linear: forward, weight-gradient and
// input-gradient steps expressed as index maps over the MFMA GEMM
// (ptl_gemm.hip).  Nothing here moves data: each step is one GEMM launch
// (plus a split-K reduction where the output is too small to fill the chip)
// reading the caller's tensors in place.
//
// Batched mode stores `ns` samples back to back (sample stride = blob->dim);
// the sample index is folded into the pixel axis of the GEMM for forward and
// input gradient, and into the contraction axis for the weight gradient, so
// the sum over samples happens in the fp32 accumulator.
#include "ptl_common.hpp"
#include "ptl_host.hpp"
#include "ptl_conv_tile.hpp"

#define STEP_BW_BOTH 3  // weight and input gradient together (library-internal step code)
#include "ptl_api.h"
#include "ptl_internal.h"

#include <stdio.h>

namespace ptl {

// ---- small kernels -----------------------------------------------------------

// Zero-stuffed copy of an output gradient for strided convolutions:
// dst[b][c][ho*sh][wo*sw] = src[b][c][ho][wo] (CHW) or the HWC equivalent.
// One workgroup per plane (CHW: a channel of a sample, HWC: a sample): it clears the plane, then scatters the
// source elements into it (one division per source element instead of five per destination element).
template <typename T>
__global__ __launch_bounds__(256) void dilate_kernel(const T *__restrict__ src, T *__restrict__ dst, int Ho, int Wo,
                                                     int Hd, int Wd, int sh, int sw, int cin) {
    // cin = innermost channel count (1 for CHW planes, C for HWC)
    const unsigned n = (unsigned)Hd * Wd * cin, m = (unsigned)Ho * Wo * cin, rowlen = (unsigned)Wo * cin;
    const T *sp = src + (size_t)blockIdx.x * m;
    T *dp = dst + (size_t)blockIdx.x * n;
    for (unsigned i = threadIdx.x; i < n; i += 256) dp[i] = (T)0;
    __syncthreads();  // orders the two writes of a position within the workgroup
    for (unsigned i = threadIdx.x; i < m; i += 256) {
        const unsigned ho = i / rowlen, r = i - ho * rowlen;
        const unsigned wo = cin == 1 ? r : r / cin, c = cin == 1 ? 0 : r - wo * cin;
        dp[((ho * sh) * Wd + wo * sw) * cin + c] = sp[i];
    }
}

// dst[0 .. n) = 0, 16 bytes per thread where the alignment allows.
template <typename T>
__global__ __launch_bounds__(256) void zero_kernel(T *__restrict__ dst, size_t n, int vec) {
    constexpr int VEC = 16 / (int)sizeof(T);
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (vec) {
        if (i * VEC + VEC <= n) reinterpret_cast<uint4 *>(dst)[i] = make_uint4(0, 0, 0, 0);
        else
            for (size_t e = i * VEC; e < n; ++e) dst[e] = (T)0;
    } else if (i < n) {
        dst[i] = (T)0;
    }
}

// out[b][c][pix] += bias[c] (CHW) or out[b][pix][c] += bias[c] (HWC)
template <typename T>
__global__ __launch_bounds__(256) void bias_add_kernel(T *__restrict__ out, const T *__restrict__ bias, size_t total,
                                                       int C, int inner) {
    size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= total) return;
    int c = (int)((idx / inner) % C);
    out[idx] = (T)((float)out[idx] + (float)bias[c]);
}

// bias_diff[c] = sum over samples and pixels of dY; one workgroup per channel.
template <typename T>
__global__ __launch_bounds__(256) void bias_grad_kernel(const T *__restrict__ dy, T *__restrict__ db, int ns, int C,
                                                        int pix, int hwc) {
    int c = blockIdx.x;
    float s = 0.f;
    size_t n = (size_t)ns * pix;
    for (size_t i = threadIdx.x; i < n; i += 256) {
        size_t b = i / pix, p = i % pix;
        size_t off = hwc ? ((b * pix + p) * C + c) : ((b * C + c) * pix + p);
        s += (float)dy[off];
    }
    __shared__ float red[256];
    red[threadIdx.x] = s;
    __syncthreads();
    for (int o = 128; o > 0; o >>= 1) {
        if ((int)threadIdx.x < o) red[threadIdx.x] += red[threadIdx.x + o];
        __syncthreads();
    }
    if (threadIdx.x == 0) db[c] = (T)red[0];
}

static inline unsigned blocks_for(size_t n) { return (unsigned)((n + 255) / 256); }

static bool fits_int(size_t v) { return v < ((size_t)1 << 31); }

// ---- Conv2D ----------------------------------------------------------------------

struct ConvGeom {
    int Ci, H, W, Co, Ho, Wo, Hk, Wk;
    int Up, Dp, Lp, Rp, sh, sw;
    int hwc;
};

template <typename Args>
static int conv_geom(const Args *a, ConvGeom &g, const char *fn, bool need_divisible) {
    if (!a || !a->input || !a->coeff || !a->output) {
        printf("[%s:] null argument structure\n", fn);
        set_error("%s: null argument structure", fn);
        return 1;
    }
    g.Ci = a->input->C;
    g.H = a->input->H;
    g.W = a->input->W;
    g.Co = a->output->C;
    g.Ho = a->output->H;
    g.Wo = a->output->W;
    g.Hk = a->coeff->H;
    g.Wk = a->coeff->W;
    g.Up = a->Upad;
    g.Dp = a->Dpad;
    g.Lp = a->Lpad;
    g.Rp = a->Rpad;
    g.sh = a->stride_h;
    g.sw = a->stride_w;
    g.hwc = a->HWC;
    if (a->USE_IM2COL != 0 && a->USE_IM2COL != 1) {
        printf("[%s:] Invalid selection of the conv2d algorithm (im2col or not)\n", fn);
        set_error("%s: USE_IM2COL must be 0 or 1", fn);
        return 1;
    }
    if (g.hwc != 0 && g.hwc != 1) {
        printf("[%s:] Invalid data layout format (HWC or CHW)!\n", fn);
        set_error("%s: HWC must be 0 or 1", fn);
        return 1;
    }
    if (a->USE_IM2COL == 0 && g.hwc == 1) {
        printf("[%s:] Naive kernel for HWC Conv2D not implemented!\n", fn);
        set_error("%s: naive HWC Conv2D does not exist in the reference", fn);
        return 1;
    }
    if (g.Ci <= 0 || g.H <= 0 || g.W <= 0 || g.Co <= 0 || g.Hk <= 0 || g.Wk <= 0 || g.sh <= 0 || g.sw <= 0 ||
        g.Up < 0 || g.Dp < 0 || g.Lp < 0 || g.Rp < 0) {
        printf("[%s:] invalid tensor geometry\n", fn);
        set_error("%s: invalid tensor geometry", fn);
        return 1;
    }
    int nh = g.H - g.Hk + g.Up + g.Dp, nw = g.W - g.Wk + g.Lp + g.Rp;
    if (nh < 0 || nw < 0) {
        printf("[%s:] kernel larger than padded input\n", fn);
        set_error("%s: kernel larger than padded input", fn);
        return 1;
    }
    if (need_divisible && a->USE_IM2COL == 1) {
        if ((nh + g.sh) % g.sh > 0) {
            printf("\n[pulp_im2col] Invalid H stride (non multiple H sizes): have H_in=%d, H_ker=%d, U_pad=%d, "
                   "D_pad=%d, H_stride=%d, remainder=%d",
                   g.H, g.Hk, g.Up, g.Dp, g.sh, (nh + g.sh) % g.sh);
            set_error("%s: H stride does not divide the padded extent", fn);
            return 1;
        }
        if ((nw + g.sw) % g.sw > 0) {
            printf("\n[pulp_im2col] Invalid W stride (non multiple W sizes): have W_in=%d, W_ker=%d, L_pad=%d, "
                   "R_pad=%d, W_stride=%d, remainder=%d",
                   g.W, g.Wk, g.Lp, g.Rp, g.sw, (nw + g.sw) % g.sw);
            set_error("%s: W stride does not divide the padded extent", fn);
            return 1;
        }
    }
    if (g.Ho != nh / g.sh + 1 || g.Wo != nw / g.sw + 1) {
        printf("[%s:] output blob is %dx%d but the geometry gives %dx%d\n", fn, g.Ho, g.Wo, nh / g.sh + 1,
               nw / g.sw + 1);
        set_error("%s: output blob size does not match the convolution geometry", fn);
        return 1;
    }
    if (g.H >= HW_LIMIT || g.W >= HW_LIMIT || g.Hk >= HW_LIMIT || g.Wk >= HW_LIMIT) {
        set_error("%s: spatial extent above %d is not supported", fn, HW_LIMIT);
        return 1;
    }
    return 0;
}

// Patch axis over output pixels (sample, ho, wo) and over kernel taps.
static AxisMap pix_axis(const ConvGeom &g, int ns) {
    AxisMap a = {};
    a.n = ns * g.Ho * g.Wo;
    a.d1 = g.Ho;
    a.d0 = g.Wo;
    if (!g.hwc) {
        a.o2 = g.Ci * g.H * g.W;
        a.o1 = g.sh * g.W;
        a.o0 = g.sw;
        a.ob = -g.Up * g.W - g.Lp;
    } else {
        a.o2 = g.H * g.W * g.Ci;
        a.o1 = g.sh * g.W * g.Ci;
        a.o0 = g.sw * g.Ci;
        a.ob = (-g.Up * g.W - g.Lp) * g.Ci;
    }
    a.h1 = g.sh;
    a.hb = -g.Up;
    a.w0 = g.sw;
    a.wb = -g.Lp;
    return a;
}

static AxisMap tap_axis(const ConvGeom &g) {
    AxisMap a = {};
    a.n = g.Ci * g.Hk * g.Wk;
    if (!g.hwc) {  // (ci, hk, wk)
        a.d1 = g.Hk;
        a.d0 = g.Wk;
        a.o2 = g.H * g.W;
        a.o1 = g.W;
        a.o0 = 1;
        a.h1 = 1;
        a.w0 = 1;
    } else {  // (hk, wk, ci)
        a.d1 = g.Wk;
        a.d0 = g.Ci;
        a.o2 = g.W * g.Ci;
        a.o1 = g.Ci;
        a.o0 = 1;
        a.h2 = 1;
        a.w1 = 1;
    }
    return a;
}

template <typename T, typename Args>
static int conv2d_fw(const Args *a, int ns, const char *fn) {
    ConvGeom g;
    if (int rc = conv_geom(a, g, fn, true)) return rc;
    if (ns <= 0) return 0;
    if (!ensure_init()) return 2;
    const int K = g.Ci * g.Hk * g.Wk, P = g.Ho * g.Wo;
    size_t in_n = (size_t)ns * g.Ci * g.H * g.W, out_n = (size_t)ns * g.Co * P;
    if (!fits_int(in_n) || !fits_int(out_n)) {
        set_error("%s: tensor larger than 2^31 elements", fn);
        return 1;
    }
    Stager sg;
    const T *X = sg.in(reinterpret_cast<const T *>(a->input->data), in_n);
    const T *Wt = sg.in(reinterpret_cast<const T *>(a->coeff->data), (size_t)g.Co * K);
    T *Y = sg.out(reinterpret_cast<T *>(a->output->data), out_n);
    const T *bias = nullptr;
    if (a->USE_BIASES == 1) {
        if (!a->bias) {
            set_error("%s: USE_BIASES=1 with a null bias blob", fn);
            return 1;
        }
        bias = sg.in(reinterpret_cast<const T *>(a->bias->data), (size_t)g.Co);
    }
    if (sg.failed()) return 2;

    int rc = -1;
    state().last_conv_direct = 0;
    state().last_conv_resident = 0;
    if (state().gemm_path != 1) {
        ConvTileDesc d = {};
        d.batch = ns; d.Cin = g.Ci; d.Hin = g.H; d.Win = g.W;
        d.Cout = g.Co; d.Ho = g.Ho; d.Wo = g.Wo;
        d.KH = g.Hk; d.KW = g.Wk; d.sh = g.sh; d.sw = g.sw;
        d.padU = g.Up; d.padD = g.Dp; d.padL = g.Lp; d.padR = g.Rp;
        d.x_sb = (long long)g.Ci * g.H * g.W; d.x_sc = (long long)g.H * g.W; d.x_sy = g.W;
        OutMap c;
        if (!g.hwc) {
            d.w_base = 0; d.w_sm = K; d.w_sc = g.Hk * g.Wk; d.w_sy = g.Wk; d.w_sx = 1;
            c.n = axis_two(ns * P, P, g.Co * P, 1);
            c.m = axis_plain(g.Co, P);
        } else {  // X[b][h][w][ci], W[co][hk][wk][ci], Y[b][pix][co]
            d.in_hwc = 1;
            d.w_base = 0; d.w_sm = K; d.w_sc = 1; d.w_sy = g.Wk * g.Ci; d.w_sx = g.Ci;
            c.n = axis_plain(ns * P, g.Co);
            c.m = axis_plain(g.Co, 1);
        }
        if (!g.hwc) rc = conv_small<T>(d, X, Wt, Y);
        // (a normalisation to apply on the way in is the small-layer kernel's business alone: nothing was launched)
        if (rc == CONV_PRE_REFUSED || conv_small_pre_pending()) return CONV_PRE_REFUSED;
        if (rc < 0) rc = conv_taps<T>(d, X, Wt, Y, c);
        if (rc < 0) rc = conv_tile<T>(d, X, Wt, Y, c);
        if (rc > 0) return sg.finish(rc);
        if (rc == 0) state().last_conv_direct = 1;
    }
    GemmArgs q = {};
    q.K = K;
    OperandMap wmap = {}, pmap = {};
    wmap.row = axis_plain(g.Co, K);
    wmap.k = axis_plain(K, 1);
    wmap.HL = wmap.WL = 1;
    pmap.row = pix_axis(g, ns);
    pmap.k = tap_axis(g);
    pmap.HL = g.H;
    pmap.WL = g.W;
    if (!g.hwc) {  // Y[b][co][pix]
        q.A = Wt;
        q.B = X;
        q.N = g.Co;
        q.M = ns * P;
        q.a = wmap;
        q.b = pmap;
        q.c.n = axis_plain(g.Co, P);
        q.c.m = axis_two(q.M, P, g.Co * P, 1);
    } else {  // Y[b][pix][co]
        q.A = X;
        q.B = Wt;
        q.N = ns * P;
        q.M = g.Co;
        q.a = pmap;
        q.b = wmap;
        q.c.n = axis_plain(q.N, g.Co);
        q.c.m = axis_plain(g.Co, 1);
    }
    q.C = Y;
    if (rc < 0) rc = gemm<T>(q);
    if (rc == 0 && bias) {
        hipLaunchKernelGGL((bias_add_kernel<T>), dim3(blocks_for(out_n)), dim3(256), 0, state().stream, Y, bias,
                           out_n, g.Co, g.hwc ? 1 : P);
        if (!hip_ok(hipGetLastError(), "bias add launch")) rc = 2;
    }
    return sg.finish(rc);
}

template <typename T, typename Args>
static int conv2d_wg(const Args *a, int ns, const char *fn) {
    ConvGeom g;
    if (int rc = conv_geom(a, g, fn, true)) return rc;
    if (ns <= 0) return 0;
    if (!ensure_init()) return 2;
    const int K = g.Ci * g.Hk * g.Wk, P = g.Ho * g.Wo;
    size_t in_n = (size_t)ns * g.Ci * g.H * g.W, out_n = (size_t)ns * g.Co * P;
    if (!fits_int(in_n) || !fits_int(out_n)) {
        set_error("%s: tensor larger than 2^31 elements", fn);
        return 1;
    }
    Stager sg;
    const T *X = sg.in(reinterpret_cast<const T *>(a->input->data), in_n);
    const T *dY = sg.in(reinterpret_cast<const T *>(a->output->diff), out_n);
    T *dW = sg.out(reinterpret_cast<T *>(a->coeff->diff), (size_t)g.Co * K);
    T *db = nullptr;
    if (a->USE_BIASES == 1) {
        if (!a->bias) {
            set_error("%s: USE_BIASES=1 with a null bias blob", fn);
            return 1;
        }
        db = sg.out(reinterpret_cast<T *>(a->bias->diff), (size_t)g.Co);
    }
    if (sg.failed()) return 2;

    int rc = -1;
    state().last_conv_direct = 0;
    state().last_conv_resident = 0;
    if (state().gemm_path != 1) {
        ConvTileDesc d = {};
        d.in_hwc = g.hwc ? 1 : 0;
        d.batch = ns; d.Cin = g.Ci; d.Hin = g.H; d.Win = g.W;
        d.Cout = g.Co; d.Ho = g.Ho; d.Wo = g.Wo;
        d.KH = g.Hk; d.KW = g.Wk; d.sh = g.sh; d.sw = g.sw;
        d.padU = g.Up; d.padD = g.Dp; d.padL = g.Lp; d.padR = g.Rp;
        d.x_sb = (long long)g.Ci * g.H * g.W; d.x_sc = (long long)g.H * g.W; d.x_sy = g.W;
        // the kernel with resident channel-blocked tiles where it is preferred; else the resident output tile kernel,
        // else (or on request) the sum over taps.  From 256 channels on either side and 16384 output pixels the sum
        // over taps goes before the output tile kernel (measured: 81 against 91 us for 256 -> 256 on 14x14 at batch
        // 128, 455 against 533 us on 28x28 at batch 256; at batch 8 the output tile kernel takes 26 against 34 us)
        const bool taps_first = d.Cin >= 128 && d.Cout >= 128 && (d.Cin >= 256 || d.Cout >= 256) &&
                                (long long)ns * g.Ho * g.Wo >= 16384;
        if (g.hwc) {  // channel-minor tensors: the sum over taps from 64 channels on, else the gathering GEMM below
            rc = conv_taps_wg<T>(d, X, dY, dW);
        } else if ((rc = conv_small_wg<T>(d, X, dY, dW,
                                           static_cast<const void *>(dW) == static_cast<const void *>(a->coeff->diff))) >= 0) {
            // (small 3x3 layers: one launch for the partial sums over sample ranges, one to add them)
        } else {
            const bool tiles_resident = sizeof(T) == 2 && state().gemm_path == 0 && conv_halo_wg_preferred(d);
            if (state().gemm_path == 3 || state().gemm_path == 5 || tiles_resident || (taps_first && state().gemm_path != 2))
                rc = conv_taps_wg<T>(d, X, dY, dW);
            if (rc < 0) rc = conv_tile_wg<T>(d, X, dY, dW);
            if (rc < 0 && state().gemm_path != 3) rc = conv_taps_wg<T>(d, X, dY, dW);
        }
        if (rc > 0) return sg.finish(rc);
        if (rc == 0) state().last_conv_direct = 1;
    }
    GemmArgs q = {};
    q.A = dY;
    q.B = X;
    q.C = dW;
    q.N = g.Co;
    q.M = K;
    q.K = ns * P;
    if (!g.hwc) {
        q.a.row = axis_plain(g.Co, P);
        q.a.k = axis_two(q.K, P, g.Co * P, 1);
    } else {
        q.a.row = axis_plain(g.Co, 1);
        q.a.k = axis_plain(q.K, g.Co);
    }
    q.a.HL = q.a.WL = 1;
    q.b.row = tap_axis(g);
    q.b.k = pix_axis(g, ns);
    q.b.HL = g.H;
    q.b.WL = g.W;
    q.c.n = axis_plain(g.Co, K);
    q.c.m = axis_plain(K, 1);
    if (rc < 0) rc = gemm<T>(q);
    if (rc == 0 && db) {
        hipLaunchKernelGGL((bias_grad_kernel<T>), dim3(g.Co), dim3(256), 0, state().stream, dY, db, ns, g.Co, P,
                           g.hwc);
        if (!hip_ok(hipGetLastError(), "bias grad launch")) rc = 2;
    }
    return sg.finish(rc);
}

template <typename T, typename Args>
static int conv2d_ig(const Args *a, int ns, const char *fn) {
    ConvGeom g;
    if (int rc = conv_geom(a, g, fn, false)) return rc;
    if (ns <= 0) return 0;
    if (!ensure_init()) return 2;
    const int Pk = g.Hk * g.Wk, K = g.Co * Pk, P = g.Ho * g.Wo;
    size_t in_n = (size_t)ns * g.Ci * g.H * g.W, out_n = (size_t)ns * g.Co * P;
    const int Hd = (g.Ho - 1) * g.sh + 1, Wd = (g.Wo - 1) * g.sw + 1;
    size_t dil_n = (size_t)ns * g.Co * Hd * Wd;
    if (!fits_int(in_n) || !fits_int(out_n) || !fits_int(dil_n)) {
        set_error("%s: tensor larger than 2^31 elements", fn);
        return 1;
    }
    Stager sg;
    const T *Wt = sg.in(reinterpret_cast<const T *>(a->coeff->data), (size_t)g.Co * g.Ci * Pk);
    const T *dY = sg.in(reinterpret_cast<const T *>(a->output->diff), out_n);
    T *dX = sg.out(reinterpret_cast<T *>(a->input->diff), in_n);
    if (sg.failed()) return 2;

    // A strided single-tap layer without padding (projection shortcut): only the input positions the layer read
    // get a gradient, dX[ci][sh*u][sw*v] = sum_co W[co][ci] dY[co][u][v] - one plain product written through a
    // strided output map into the zeroed tensor (the general route below would run a stride-1 pass over a
    // zero-stuffed gradient four times the size: measured 32 against 11 us for 16 -> 32 channels, 32x32, batch 128).
    // With bottom / right padding the last output rows or columns sit on padded positions outside the input;
    // the scatter map has no coordinate test, so such geometries take the general route below.
    const bool taps_inside = (long long)(g.Ho - 1) * g.sh < g.H && (long long)(g.Wo - 1) * g.sw < g.W;
    if (Pk == 1 && (g.sh != 1 || g.sw != 1) && g.Up == 0 && g.Lp == 0 && taps_inside && state().gemm_path != 1) {
        const int vec = reinterpret_cast<uintptr_t>(dX) % 16 == 0;
        const size_t threads = vec ? (in_n + 16 / sizeof(T) - 1) / (16 / sizeof(T)) : in_n;
        hipLaunchKernelGGL((zero_kernel<T>), dim3(blocks_for(threads)), dim3(256), 0, state().stream, dX, in_n, vec);
        if (!hip_ok(hipGetLastError(), "zero launch")) return sg.finish(2);
        state().last_conv_direct = 0;
        GemmArgs q = {};
        q.K = g.Co;
        q.C = dX;
        q.a.HL = q.a.WL = q.b.HL = q.b.WL = 1;
        AxisMap pix = {};  // output pixel (sample, u, v) inside the input tensor
        pix.n = ns * P;
        pix.d1 = g.Ho;
        pix.d0 = g.Wo;
        if (!g.hwc) {
            q.A = Wt;
            q.B = dY;
            q.N = g.Ci;
            q.M = ns * P;
            q.a.row = axis_plain(g.Ci, 1);
            q.a.k = axis_plain(g.Co, g.Ci);
            q.b.row = axis_two(q.M, P, g.Co * P, 1);
            q.b.k = axis_plain(g.Co, P);
            pix.o2 = g.Ci * g.H * g.W;
            pix.o1 = g.sh * g.W;
            pix.o0 = g.sw;
            q.c.n = axis_plain(g.Ci, g.H * g.W);
            q.c.m = pix;
        } else {
            q.A = dY;
            q.B = Wt;
            q.N = ns * P;
            q.M = g.Ci;
            q.a.row = axis_plain(q.N, g.Co);
            q.a.k = axis_plain(g.Co, 1);
            q.b.row = axis_plain(g.Ci, 1);
            q.b.k = axis_plain(g.Co, g.Ci);
            pix.o2 = g.H * g.W * g.Ci;
            pix.o1 = g.sh * g.W * g.Ci;
            pix.o0 = g.sw * g.Ci;
            q.c.n = pix;
            q.c.m = axis_plain(g.Ci, 1);
        }
        return sg.finish(gemm<T>(q));
    }

    // Small stride-2 layers (3x3 or 1x1): the small-layer kernel stuffs the zeros while it fills its LDS tile.
    if (!g.hwc && g.sh == 2 && g.sw == 2 && g.Hk == g.Wk && (g.Hk == 3 || g.Hk == 1)) {
        ConvTileDesc d = {};
        d.batch = ns; d.Cin = g.Co; d.Hin = g.Ho; d.Win = g.Wo; d.in_dil = 2;
        d.Cout = g.Ci; d.Ho = g.H; d.Wo = g.W;
        d.KH = g.Hk; d.KW = g.Wk; d.sh = 1; d.sw = 1;
        d.padU = g.Hk - 1 - g.Up; d.padL = g.Wk - 1 - g.Lp;
        d.padD = g.H + g.Hk - 1 - Hd - d.padU; d.padR = g.W + g.Wk - 1 - Wd - d.padL;
        d.x_sb = (long long)g.Co * P; d.x_sc = P; d.x_sy = g.Wo;
        d.w_base = Pk - 1; d.w_sm = Pk; d.w_sc = g.Ci * Pk; d.w_sy = -g.Wk; d.w_sx = -1;
        state().last_conv_direct = 0;
        state().last_conv_resident = 0;
        const int rc = conv_small<T>(d, dY, Wt, dX);
        if (rc == 0) state().last_conv_direct = 1;
        if (rc >= 0) return sg.finish(rc);
    }

    // A strided forward is undone by a unit-stride pass over the zero-stuffed gradient.
    if (g.sh != 1 || g.sw != 1) {
        T *dil = static_cast<T *>(scratch(dil_n * sizeof(T)));
        if (!dil) return 2;
        hipLaunchKernelGGL((dilate_kernel<T>), dim3((unsigned)(g.hwc ? ns : ns * g.Co)), dim3(256), 0, state().stream, dY,
                           dil, g.Ho, g.Wo, Hd, Wd, g.sh, g.sw, g.hwc ? g.Co : 1);
        if (!hip_ok(hipGetLastError(), "dilate launch")) return sg.finish(2);
        dY = dil;
    }

    // dX[ci,hi,wi] = sum_{co,hk,wk} W[co,ci,hk,wk] * dYd[co, hi+Up-hk, wi+Lp-wk]
    OperandMap wmap = {}, gmap = {};
    wmap.HL = wmap.WL = 1;
    gmap.HL = Hd;
    gmap.WL = Wd;
    gmap.row.n = ns * g.H * g.W;
    gmap.row.d1 = g.H;
    gmap.row.d0 = g.W;
    gmap.row.h1 = 1;
    gmap.row.hb = g.Up;
    gmap.row.w0 = 1;
    gmap.row.wb = g.Lp;
    gmap.k.n = K;
    state().last_conv_direct = 0;
    state().last_conv_resident = 0;
    if (state().gemm_path != 1) {
        ConvTileDesc d = {};
        d.batch = ns; d.Cin = g.Co; d.Hin = Hd; d.Win = Wd;
        d.Cout = g.Ci; d.Ho = g.H; d.Wo = g.W;
        d.KH = g.Hk; d.KW = g.Wk; d.sh = 1; d.sw = 1;
        d.padU = g.Hk - 1 - g.Up; d.padL = g.Wk - 1 - g.Lp;
        d.padD = g.H + g.Hk - 1 - Hd - d.padU; d.padR = g.W + g.Wk - 1 - Wd - d.padL;
        d.x_sb = (long long)g.Co * Hd * Wd; d.x_sc = (long long)Hd * Wd; d.x_sy = Wd;
        OutMap c;
        if (!g.hwc) {
            d.w_base = Pk - 1; d.w_sm = Pk; d.w_sc = g.Ci * Pk; d.w_sy = -g.Wk; d.w_sx = -1;
            c.n = axis_two(ns * g.H * g.W, g.H * g.W, g.Ci * g.H * g.W, 1);
            c.m = axis_plain(g.Ci, g.H * g.W);
        } else {  // dY[b][pix][co], W[co][hk][wk][ci], dX[b][pix][ci]
            d.in_hwc = 1;
            d.w_base = (Pk - 1) * g.Ci; d.w_sm = 1; d.w_sc = Pk * g.Ci; d.w_sy = -g.Wk * g.Ci; d.w_sx = -g.Ci;
            c.n = axis_plain(ns * g.H * g.W, g.Ci);
            c.m = axis_plain(g.Ci, 1);
        }
        // (the zero-stuffed gradient of a strided layer lives in the scratch buffer the tap route would reuse)
        int rc = !g.hwc ? conv_small<T>(d, dY, Wt, dX) : -1;
        if (rc < 0 && g.sh == 1 && g.sw == 1) rc = conv_taps<T>(d, dY, Wt, dX, c);
        if (rc < 0) rc = conv_tile<T>(d, dY, Wt, dX, c);
        if (rc == 0) state().last_conv_direct = 1;
        if (rc >= 0) return sg.finish(rc);
    }
    GemmArgs q = {};
    q.K = K;
    q.C = dX;
    if (!g.hwc) {
        wmap.row = axis_plain(g.Ci, Pk);
        wmap.k = axis_two(K, Pk, g.Ci * Pk, 1);  // (co, tap)
        gmap.row.o2 = g.Co * Hd * Wd;
        gmap.row.o1 = Wd;
        gmap.row.o0 = 1;
        gmap.row.ob = g.Up * Wd + g.Lp;
        gmap.k.d1 = g.Hk;  // (co, hk, wk)
        gmap.k.d0 = g.Wk;
        gmap.k.o2 = Hd * Wd;
        gmap.k.o1 = -Wd;
        gmap.k.o0 = -1;
        gmap.k.h1 = -1;
        gmap.k.w0 = -1;
        q.A = Wt;
        q.B = dY;
        q.N = g.Ci;
        q.M = ns * g.H * g.W;
        q.a = wmap;
        q.b = gmap;
        q.c.n = axis_plain(g.Ci, g.H * g.W);
        q.c.m = axis_two(q.M, g.H * g.W, g.Ci * g.H * g.W, 1);
    } else {
        // contraction index (hk, wk, co); weights are [co][hk][wk][ci]
        wmap.row = axis_plain(g.Ci, 1);
        wmap.k.n = K;
        wmap.k.d1 = g.Wk;
        wmap.k.d0 = g.Co;
        wmap.k.o2 = g.Wk * g.Ci;
        wmap.k.o1 = g.Ci;
        wmap.k.o0 = Pk * g.Ci;
        gmap.row.o2 = Hd * Wd * g.Co;
        gmap.row.o1 = Wd * g.Co;
        gmap.row.o0 = g.Co;
        gmap.row.ob = (g.Up * Wd + g.Lp) * g.Co;
        gmap.k.d1 = g.Wk;
        gmap.k.d0 = g.Co;
        gmap.k.o2 = -Wd * g.Co;
        gmap.k.o1 = -g.Co;
        gmap.k.o0 = 1;
        gmap.k.h2 = -1;
        gmap.k.w1 = -1;
        q.A = dY;
        q.B = Wt;
        q.N = ns * g.H * g.W;
        q.M = g.Ci;
        q.a = gmap;
        q.b = wmap;
        q.c.n = axis_plain(q.N, g.Ci);
        q.c.m = axis_plain(g.Ci, 1);
    }
    return sg.finish(gemm<T>(q));
}

// ---- Pointwise convolution ------------------------------------------------------------
// CHW: X[b][Ci][HW], W[Co][Ci], Y[b][Co][HW].
// HWC: X[b][HW][Ci], Y[b][HW][Co]; weights are [Ci][Co] in the fp32 layer
// (lib/sources/pulp_conv_pw_fp32.c:67-74) and [Co][Ci] in the fp16 layer
// (lib/sources/pulp_conv_pw_fp16.c:70-76).

template <typename Args>
static int pw_geom(const Args *a, const char *fn) {
    if (!a || !a->input || !a->coeff || !a->output) {
        printf("[%s] null argument structure\n", fn);
        set_error("%s: null argument structure", fn);
        return 1;
    }
    if (a->HWC != 0 && a->HWC != 1) {
        printf("[%s] Invalid HWC parameter!\n", fn);
        set_error("%s: HWC must be 0 or 1", fn);
        return 1;
    }
    if (a->input->C <= 0 || a->output->C <= 0 || a->input->H <= 0 || a->input->W <= 0 ||
        a->input->H != a->output->H || a->input->W != a->output->W) {
        printf("[%s] invalid tensor geometry\n", fn);
        set_error("%s: invalid tensor geometry", fn);
        return 1;
    }
    return 0;
}

// Weight and input gradient of one call (the batched twin of pulp_conv2d_*_bw_cl): honours skip_wg_grad /
// skip_in_grad; where both run on the resident-tile kernels they share the blocked copy of the output gradient.
template <typename T, typename Args>
static int conv2d_bw(const Args *a, int ns, const char *fn) {
    if (!a) {
        set_error("%s: null argument structure", fn);
        return 1;
    }
    const bool wg = a->skip_wg_grad == 0, ig = a->skip_in_grad == 0;
    if (wg && ig && a->USE_BIASES != 1 && ns >= 1 && a->input && a->coeff && a->output) {
        ConvGeom g;
        if (int rc = conv_geom(a, g, fn, true)) return rc;
        const int P = g.Ho * g.Wo, Pk = g.Hk * g.Wk, K = g.Ci * Pk;
        size_t in_n = (size_t)ns * g.Ci * g.H * g.W, out_n = (size_t)ns * g.Co * P;
        const bool unit = g.sh == 1 && g.sw == 1 && g.Up + g.Dp == g.Hk - 1 && g.Lp + g.Rp == g.Wk - 1;
        const bool halving = g.sh == 2 && g.sw == 2;  // (small layers only: the zeros are stuffed on the way into LDS)
        if (!g.hwc && g.Hk == g.Wk && (g.Hk == 3 || g.Hk == 1) && (unit || halving) && fits_int(in_n) && fits_int(out_n) &&
            (state().gemm_path == 0 || state().gemm_path == 5 || state().gemm_path == 6)) {
            if (!ensure_init()) return 2;
            ConvTileDesc f = {}, b = {};
            f.batch = ns; f.Cin = g.Ci; f.Hin = g.H; f.Win = g.W;
            f.Cout = g.Co; f.Ho = g.Ho; f.Wo = g.Wo;
            f.KH = g.Hk; f.KW = g.Wk; f.sh = g.sh; f.sw = g.sw;
            f.padU = g.Up; f.padD = g.Dp; f.padL = g.Lp; f.padR = g.Rp;
            f.x_sb = (long long)g.Ci * g.H * g.W; f.x_sc = (long long)g.H * g.W; f.x_sy = g.W;
            // the input gradient: a unit-stride pass over the output gradient, zero-stuffed where the forward strode
            const int Hd = (g.Ho - 1) * g.sh + 1, Wd = (g.Wo - 1) * g.sw + 1;
            b.batch = ns; b.Cin = g.Co; b.Hin = g.Ho; b.Win = g.Wo; b.in_dil = halving ? 2 : 0;
            b.Cout = g.Ci; b.Ho = g.H; b.Wo = g.W;
            b.KH = g.Hk; b.KW = g.Wk; b.sh = 1; b.sw = 1;
            b.padU = g.Hk - 1 - g.Up; b.padL = g.Wk - 1 - g.Lp;
            b.padD = g.H + g.Hk - 1 - Hd - b.padU; b.padR = g.W + g.Wk - 1 - Wd - b.padL;
            b.x_sb = (long long)g.Co * P; b.x_sc = P; b.x_sy = g.Wo;
            b.w_base = Pk - 1; b.w_sm = Pk; b.w_sc = g.Ci * Pk; b.w_sy = -g.Wk; b.w_sx = -1;
            // small layers: both products in one launch; wide layers: one shared copy of the output gradient
            const bool small = g.Ci <= 64 && g.Co <= 64 && g.W % (16 / (int)sizeof(T)) == 0 && state().gemm_path != 5;
            const bool wide = unit && g.Hk == 3 && sizeof(T) == 2 && ns > 1 && state().gemm_path != 6 && conv_halo_wg_preferred(f);
            if (small || wide) {
                Stager sg;
                const T *X = sg.in(reinterpret_cast<const T *>(a->input->data), in_n);
                const T *dY = sg.in(reinterpret_cast<const T *>(a->output->diff), out_n);
                const T *Wt = sg.in(reinterpret_cast<const T *>(a->coeff->data), (size_t)g.Co * K);
                T *dW = sg.out(reinterpret_cast<T *>(a->coeff->diff), (size_t)g.Co * K);
                T *dX = sg.out(reinterpret_cast<T *>(a->input->diff), in_n);
                if (sg.failed()) return sg.rejected() ? 1 : 2;
                state().last_conv_direct = 0;
                state().last_conv_resident = 0;
                // (a host tensor's gradient is a staging copy that this call copies back: its sums cannot wait)
                const bool on_device = static_cast<const void *>(dW) == static_cast<const void *>(a->coeff->diff);
                int rc = small ? conv_small_bw<T>(f, b, X, dY, Wt, dW, dX, on_device) : -1;
                if (rc < 0 && wide) rc = conv_halo_bw<T>(f, b, X, dY, Wt, dW, dX);
                if (rc >= 0) {
                    if (rc == 0) state().last_conv_direct = 1;
                    return sg.finish(rc);
                }
                // neither kernel took the layer: nothing was written, so nothing of the staged gradients goes back
                // to the caller; the two single-step calls below are the only writers
                sg.discard();
            }
        }
    }
    int rc = wg ? conv2d_wg<T>(a, ns, fn) : 0;
    if (rc == 0 && ig) rc = conv2d_ig<T>(a, ns, fn);
    return rc;
}

template <typename T, typename Args>
static int pw_step(const Args *a, int ns, int step, const char *fn) {
    if (int rc = pw_geom(a, fn)) return rc;
    if (ns <= 0) return 0;
    if (!ensure_init()) return 2;
    const int Ci = a->input->C, Co = a->output->C, HW = a->input->H * a->input->W;
    const bool hwc = a->HWC == 1;
    const bool w_ci_major = hwc && sizeof(T) == 4;  // fp32 HWC stores [Ci][Co]
    const int w_co = w_ci_major ? 1 : Ci, w_ci = w_ci_major ? Co : 1;
    size_t in_n = (size_t)ns * Ci * HW, out_n = (size_t)ns * Co * HW;
    if (!fits_int(in_n) || !fits_int(out_n)) {
        set_error("%s: tensor larger than 2^31 elements", fn);
        return 1;
    }
    Stager sg;
    GemmArgs q = {};
    q.a.HL = q.a.WL = q.b.HL = q.b.WL = 1;
    const int BP = ns * HW;
    if (step == STEP_FW) {
        const T *X = sg.in(reinterpret_cast<const T *>(a->input->data), in_n);
        const T *Wt = sg.in(reinterpret_cast<const T *>(a->coeff->data), (size_t)Co * Ci);
        T *Y = sg.out(reinterpret_cast<T *>(a->output->data), out_n);
        q.C = Y;
        q.K = Ci;
        if (!hwc) {
            q.A = Wt;
            q.B = X;
            q.N = Co;
            q.M = BP;
            q.a.row = axis_plain(Co, Ci);
            q.a.k = axis_plain(Ci, 1);
            q.b.row = axis_two(BP, HW, Ci * HW, 1);
            q.b.k = axis_plain(Ci, HW);
            q.c.n = axis_plain(Co, HW);
            q.c.m = axis_two(BP, HW, Co * HW, 1);
        } else {
            q.A = X;
            q.B = Wt;
            q.N = BP;
            q.M = Co;
            q.a.row = axis_plain(BP, Ci);
            q.a.k = axis_plain(Ci, 1);
            q.b.row = axis_plain(Co, w_co);
            q.b.k = axis_plain(Ci, w_ci);
            q.c.n = axis_plain(BP, Co);
            q.c.m = axis_plain(Co, 1);
        }
    } else if (step == STEP_WGT_GRAD) {
        const T *X = sg.in(reinterpret_cast<const T *>(a->input->data), in_n);
        const T *dY = sg.in(reinterpret_cast<const T *>(a->output->diff), out_n);
        T *dW = sg.out(reinterpret_cast<T *>(a->coeff->diff), (size_t)Co * Ci);
        q.A = dY;
        q.B = X;
        q.C = dW;
        q.N = Co;
        q.M = Ci;
        q.K = BP;
        if (!hwc) {
            q.a.row = axis_plain(Co, HW);
            q.a.k = axis_two(BP, HW, Co * HW, 1);
            q.b.row = axis_plain(Ci, HW);
            q.b.k = axis_two(BP, HW, Ci * HW, 1);
        } else {
            q.a.row = axis_plain(Co, 1);
            q.a.k = axis_plain(BP, Co);
            q.b.row = axis_plain(Ci, 1);
            q.b.k = axis_plain(BP, Ci);
        }
        q.c.n = axis_plain(Co, w_co);
        q.c.m = axis_plain(Ci, w_ci);
    } else {
        const T *Wt = sg.in(reinterpret_cast<const T *>(a->coeff->data), (size_t)Co * Ci);
        const T *dY = sg.in(reinterpret_cast<const T *>(a->output->diff), out_n);
        T *dX = sg.out(reinterpret_cast<T *>(a->input->diff), in_n);
        q.C = dX;
        q.K = Co;
        if (!hwc) {
            q.A = Wt;
            q.B = dY;
            q.N = Ci;
            q.M = BP;
            q.a.row = axis_plain(Ci, w_ci);
            q.a.k = axis_plain(Co, w_co);
            q.b.row = axis_two(BP, HW, Co * HW, 1);
            q.b.k = axis_plain(Co, HW);
            q.c.n = axis_plain(Ci, HW);
            q.c.m = axis_two(BP, HW, Ci * HW, 1);
        } else {
            q.A = dY;
            q.B = Wt;
            q.N = BP;
            q.M = Ci;
            q.a.row = axis_plain(BP, Co);
            q.a.k = axis_plain(Co, 1);
            q.b.row = axis_plain(Ci, w_ci);
            q.b.k = axis_plain(Co, w_co);
            q.c.n = axis_plain(BP, Ci);
            q.c.m = axis_plain(Ci, 1);
        }
    }
    if (sg.failed()) return 2;
    return sg.finish(gemm<T>(q));
}

// ---- Linear --------------------------------------------------------------------------
// W is [out][in] row-major (lib/sources/pulp_linear_fp32.c:39-46); sample b of
// the input/output blobs is a vector of blob->dim elements.

template <typename T>
__global__ __launch_bounds__(256) void rowvec_add_kernel(T *__restrict__ y, const T *__restrict__ b, size_t total,
                                                         int dim) {
    size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= total) return;
    y[idx] = (T)((float)y[idx] + (float)b[idx % dim]);
}

template <typename T, typename Args>
static int linear_step(const Args *a, int ns, int step, const char *fn) {
    if (!a || !a->input || !a->coeff || !a->output) {
        printf("[%s] null argument structure\n", fn);
        set_error("%s: null argument structure", fn);
        return 1;
    }
    const int in = a->input->dim, out = a->output->dim;
    if (in <= 0 || out <= 0) {
        printf("[%s] invalid tensor geometry\n", fn);
        set_error("%s: invalid tensor geometry", fn);
        return 1;
    }
    if (ns <= 0) return 0;
    if (!ensure_init()) return 2;
    if (!fits_int((size_t)ns * in) || !fits_int((size_t)ns * out) || !fits_int((size_t)in * out)) {
        set_error("%s: tensor larger than 2^31 elements", fn);
        return 1;
    }
    const bool use_bias = a->use_biases == 1;
    if (use_bias && !a->bias) {
        set_error("%s: use_biases=1 with a null bias blob", fn);
        return 1;
    }
    Stager sg;
    int rc = 0;
    if (step == STEP_FW) {
        const T *X = sg.in(reinterpret_cast<const T *>(a->input->data), (size_t)ns * in);
        const T *Wt = sg.in(reinterpret_cast<const T *>(a->coeff->data), (size_t)out * in);
        T *Y = sg.out(reinterpret_cast<T *>(a->output->data), (size_t)ns * out);
        const T *bias = use_bias ? sg.in(reinterpret_cast<const T *>(a->bias->data), (size_t)out) : nullptr;
        if (sg.failed()) return 2;
        if (ns == 1)
            rc = mm_dispatch<T>(Wt, X, Y, out, 1, in, 0);
        else
            rc = mm_dispatch<T>(X, Wt, Y, ns, out, in, 1);  // Y[b][o] = X[b][:] . W[o][:]
        if (rc == 0 && bias) {
            size_t total = (size_t)ns * out;
            hipLaunchKernelGGL((rowvec_add_kernel<T>), dim3(blocks_for(total)), dim3(256), 0, state().stream, Y,
                               bias, total, out);
            if (!hip_ok(hipGetLastError(), "bias add launch")) rc = 2;
        }
    } else if (step == STEP_BW_BOTH) {
        // weight and input gradient of a batch in one launch
        const T *X = sg.in(reinterpret_cast<const T *>(a->input->data), (size_t)ns * in);
        const T *Wt = sg.in(reinterpret_cast<const T *>(a->coeff->data), (size_t)out * in);
        const T *dY = sg.in(reinterpret_cast<const T *>(a->output->diff), (size_t)ns * out);
        T *dW = sg.out(reinterpret_cast<T *>(a->coeff->diff), (size_t)out * in);
        T *dX = sg.out(reinterpret_cast<T *>(a->input->diff), (size_t)ns * in);
        T *db = use_bias ? sg.out(reinterpret_cast<T *>(a->bias->diff), (size_t)out) : nullptr;
        if (sg.failed()) return 2;
        GemmArgs q = {}, r = {};
        q.A = dY;  // dW[o][i] = sum_b dY[b][o] * X[b][i]
        q.B = X;
        q.C = dW;
        q.N = out;
        q.M = in;
        q.K = ns;
        q.a.row = axis_plain(out, 1);
        q.a.k = axis_plain(ns, out);
        q.b.row = axis_plain(in, 1);
        q.b.k = axis_plain(ns, in);
        q.a.HL = q.a.WL = q.b.HL = q.b.WL = 1;
        q.c.n = axis_plain(out, in);
        q.c.m = axis_plain(in, 1);
        r.A = dY;  // dX[b][i] = sum_o dY[b][o] * W[o][i]
        r.B = Wt;
        r.C = dX;
        r.N = ns;
        r.M = in;
        r.K = out;
        r.a.row = axis_plain(ns, out);
        r.a.k = axis_plain(out, 1);
        r.b.row = axis_plain(in, 1);
        r.b.k = axis_plain(out, in);
        r.a.HL = r.a.WL = r.b.HL = r.b.WL = 1;
        r.c.n = axis_plain(ns, in);
        r.c.m = axis_plain(in, 1);
        rc = gemm_pair<T>(q, r);
        if (rc == 0 && db) {
            hipLaunchKernelGGL((bias_grad_kernel<T>), dim3(out), dim3(256), 0, state().stream, dY, db, ns, out, 1,
                               1);
            if (!hip_ok(hipGetLastError(), "bias grad launch")) rc = 2;
        }
    } else if (step == STEP_WGT_GRAD) {
        const T *X = sg.in(reinterpret_cast<const T *>(a->input->data), (size_t)ns * in);
        const T *dY = sg.in(reinterpret_cast<const T *>(a->output->diff), (size_t)ns * out);
        T *dW = sg.out(reinterpret_cast<T *>(a->coeff->diff), (size_t)out * in);
        T *db = use_bias ? sg.out(reinterpret_cast<T *>(a->bias->diff), (size_t)out) : nullptr;
        if (sg.failed()) return 2;
        if (ns == 1) {
            rc = mm_dispatch<T>(dY, X, dW, out, in, 1, 0);
        } else {  // dW[o][i] = sum_b dY[b][o] * X[b][i]
            GemmArgs q = {};
            q.A = dY;
            q.B = X;
            q.C = dW;
            q.N = out;
            q.M = in;
            q.K = ns;
            q.a.row = axis_plain(out, 1);
            q.a.k = axis_plain(ns, out);
            q.b.row = axis_plain(in, 1);
            q.b.k = axis_plain(ns, in);
            q.a.HL = q.a.WL = q.b.HL = q.b.WL = 1;
            q.c.n = axis_plain(out, in);
            q.c.m = axis_plain(in, 1);
            rc = gemm<T>(q);
        }
        if (rc == 0 && db) {  // db[o] = sum_b dY[b][o]
            hipLaunchKernelGGL((bias_grad_kernel<T>), dim3(out), dim3(256), 0, state().stream, dY, db, ns, out, 1,
                               1);
            if (!hip_ok(hipGetLastError(), "bias grad launch")) rc = 2;
        }
    } else {
        const T *Wt = sg.in(reinterpret_cast<const T *>(a->coeff->data), (size_t)out * in);
        const T *dY = sg.in(reinterpret_cast<const T *>(a->output->diff), (size_t)ns * out);
        T *dX = sg.out(reinterpret_cast<T *>(a->input->diff), (size_t)ns * in);
        if (sg.failed()) return 2;
        rc = mm_dispatch<T>(dY, Wt, dX, ns, in, out, 0);  // dX[b][i] = sum_o dY[b][o] * W[o][i]
    }
    return sg.finish(rc);
}

template <typename T>
static int bias_add_mat(T *mat, const T *bias, int N, int M, int per_row) {
    if (N <= 0 || M <= 0) return 0;
    if (!mat || !bias) {
        set_error("bias add: null argument");
        return 1;
    }
    if (!ensure_init()) return 2;
    Stager sg;
    size_t total = (size_t)N * M;
    T *m = sg.inout(mat, total);
    const T *b = sg.in(bias, (size_t)(per_row ? N : M));
    if (sg.failed()) return 2;
    hipLaunchKernelGGL((bias_add_kernel<T>), dim3(blocks_for(total)), dim3(256), 0, state().stream, m, b, total,
                       per_row ? N : M, per_row ? M : 1);
    return sg.finish(hip_ok(hipGetLastError(), "bias add launch") ? 0 : 2);
}

template <typename T>
static int rowsum_mat(const T *mat, T *out, int N, int K) {
    if (N <= 0 || K <= 0) return 0;
    if (!mat || !out) {
        set_error("row sum: null argument");
        return 1;
    }
    if (!ensure_init()) return 2;
    Stager sg;
    const T *m = sg.in(mat, (size_t)N * K);
    T *o = sg.out(out, (size_t)N);
    if (sg.failed()) return 2;
    hipLaunchKernelGGL((bias_grad_kernel<T>), dim3(N), dim3(256), 0, state().stream, m, o, 1, N, K, 0);
    return sg.finish(hip_ok(hipGetLastError(), "row sum launch") ? 0 : 2);
}

template <typename T, typename Args>
static int conv2d_fw_stats(const Args *a, int ns, ::ptl_norm_stats *st, const char *fn) {
    if (!st) {
        set_error("%s: null statistics struct", fn);
        return 1;
    }
    st->valid = 0;
    const bool take = a && a->USE_BIASES != 1;  // (a bias is added by a launch behind the kernel that forms the sums)
    if (take) conv_small_stats_to(st);
    const int rc = conv2d_fw<T>(a, ns, fn);
    conv_small_stats_to(nullptr);
    if (rc) st->valid = 0;
    return rc;
}

// The forward call of a normalisation layer and of the convolution that reads its output, in that order - as one
// launch where the small-layer kernel takes the convolution (it then applies the normalisation to its input tile while
// it loads it and writes the normalisation's output on the way), as the two calls otherwise.  Same results bit for bit.
template <typename T, typename Args, typename NormArgs, typename Fusion>
static int conv2d_fw_normed(const Args *a, int ns, ::ptl_norm_stats *st_out, const NormArgs *n, const Fusion *f,
                            const ::ptl_norm_stats *st_in, int (*norm_call)(const NormArgs *, const Fusion *,
                                                                            const ::ptl_norm_stats *),
                            const char *fn) {
    if (!a || !n) {
        set_error("%s: null argument", fn);
        return 1;
    }
    if (st_out) st_out->valid = 0;
    const bool shapes = a->input && n->input && n->output && n->output->data && n->output->data == a->input->data &&
                        n->input->data && n->weight_data && n->bias_data && n->eps && ns > 0 && n->B == ns &&
                        n->C == a->input->C && n->H == a->input->H && n->W == a->input->W && n->C > 0 && n->H > 0 && n->W > 0;
    const bool sums = st_in && st_in->valid == 1 && st_in->part && st_in->parts > 0 && shapes && st_in->channels == n->C &&
                      st_in->count == (size_t)ns * n->H * n->W &&
                      (size_t)n->C * st_in->parts * 4 * sizeof(float) <= st_in->bytes;
    if (sums && ensure_init() && state().gemm_path != 1) {
        const size_t cnt = (size_t)ns * n->C * n->H * n->W;
        bool device;
        {
            Stager sg(true);  // (host tensors: the two calls, which stage them)
            (void)sg.in(reinterpret_cast<const T *>(n->input->data), cnt);
            (void)sg.out(reinterpret_cast<T *>(n->output->data), cnt);
            if (f && f->skip) (void)sg.in(reinterpret_cast<const T *>(f->skip), cnt);
            (void)sg.in(reinterpret_cast<const T *>(n->weight_data), (size_t)n->C);
            (void)sg.in(reinterpret_cast<const T *>(n->bias_data), (size_t)n->C);
            (void)sg.in(reinterpret_cast<const T *>(n->eps), (size_t)1);
            device = !sg.failed();
        }
        if (device) {
            ConvPreNorm pre = {};
            pre.x = n->input->data;
            pre.out = n->output->data;
            pre.skip = f ? f->skip : nullptr;
            pre.weight = n->weight_data;
            pre.bias = n->bias_data;
            pre.eps = n->eps;
            pre.part = st_in->part;
            pre.parts = st_in->parts;
            pre.relu = f && f->relu ? 1 : 0;
            pre.count = st_in->count;
            conv_small_pre_to(&pre);
            const int rc = st_out ? conv2d_fw_stats<T>(a, ns, st_out, fn) : conv2d_fw<T>(a, ns, fn);
            conv_small_pre_to(nullptr);
            if (rc != CONV_PRE_REFUSED) return rc;
        }
    }
    if (int rc = norm_call(n, f, st_in)) return rc;
    return st_out ? conv2d_fw_stats<T>(a, ns, st_out, fn) : conv2d_fw<T>(a, ns, fn);
}

// Backward step whose input gradient becomes the gradient a normalisation in front of this layer starts from:
// input->diff = (dX [+ post->add]) [where post->mask > 0, else 0], rounded to T after the sum like a tensor an
// element-wise layer would have written, and the sums of that gradient and of its products with post->x in `sums`
// (valid = 1) - when the small-layer kernel takes the layer.  Any other route leaves the plain input gradient and
// sums->valid = 0.  Device tensors only.
template <typename T, typename Args>
static int conv2d_bw_post(const Args *a, int ns, ::ptl_wg_batch *batch, const ::ptl_grad_post *post,
                          ::ptl_norm_stats *sums, const char *fn) {
    if (!post || !sums || !post->x) {
        set_error("%s: null gradient epilogue or statistics struct", fn);
        return 1;
    }
    sums->valid = 0;
    if (!a || !a->input || !a->input->diff || a->skip_in_grad) {
        set_error("%s: the gradient epilogue needs the input gradient", fn);
        return 1;
    }
    if (ns <= 0 || a->input->C <= 0 || a->input->H <= 0 || a->input->W <= 0) {
        set_error("%s: invalid tensor geometry", fn);
        return 1;
    }
    if (!ensure_init()) return 2;
    const size_t n = (size_t)ns * a->input->C * a->input->H * a->input->W;
    {
        Stager sg(true);  // host tensors are rejected
        (void)sg.inout(reinterpret_cast<T *>(a->input->diff), n);
        if (post->add) (void)sg.in(reinterpret_cast<const T *>(post->add), n);
        if (post->mask) (void)sg.in(reinterpret_cast<const T *>(post->mask), n);
        (void)sg.in(reinterpret_cast<const T *>(post->x), n);
        if (sg.failed()) return sg.rejected() ? 1 : 2;
    }
    conv_small_defer_to(batch);
    conv_small_post_to(post, sums);
    const int rc = conv2d_bw<T>(a, ns, fn);
    conv_small_post_to(nullptr, nullptr);
    conv_small_defer_to(nullptr);
    if (rc) sums->valid = 0;
    return rc;
}

}  // namespace ptl

// ---- C ABI -------------------------------------------------------------------------------
using ptl::half_t;

extern "C" {

void ptl_internal_set_status(int s) { ptl::set_status(s); }
int ptl_internal_bias_add_fp32(float *mat, const float *bias, int N, int M, int per_row) {
    return ptl::bias_add_mat<float>(mat, bias, N, M, per_row);
}
int ptl_internal_bias_add_fp16(fp16 *mat, const fp16 *bias, int N, int M, int per_row) {
    return ptl::bias_add_mat<half_t>(reinterpret_cast<half_t *>(mat), reinterpret_cast<const half_t *>(bias), N, M,
                                     per_row);
}
int ptl_internal_rowsum_fp32(const float *mat, float *out, int N, int K) {
    return ptl::rowsum_mat<float>(mat, out, N, K);
}
int ptl_internal_rowsum_fp16(const fp16 *mat, fp16 *out, int N, int K) {
    return ptl::rowsum_mat<half_t>(reinterpret_cast<const half_t *>(mat), reinterpret_cast<half_t *>(out), N, K);
}

int ptl_conv2d_fp32_fw_batched(const struct Conv2D_args *a, int ns) {
    return ptl::conv2d_fw<float>(a, ns, "pulp_conv2d_fp32_fw_cl");
}
int ptl_conv2d_fp32_wg_batched(const struct Conv2D_args *a, int ns) {
    return ptl::conv2d_wg<float>(a, ns, "pulp_conv2d_fp32_bw_param_grads_cl");
}
int ptl_conv2d_fp32_ig_batched(const struct Conv2D_args *a, int ns) {
    return ptl::conv2d_ig<float>(a, ns, "pulp_conv2d_fp32_bw_input_grads_cl");
}
int ptl_conv2d_fp16_fw_batched(const struct Conv2D_args_fp16 *a, int ns) {
    return ptl::conv2d_fw<half_t>(a, ns, "pulp_conv2d_fp16_fw_cl");
}
int ptl_conv2d_fp16_wg_batched(const struct Conv2D_args_fp16 *a, int ns) {
    return ptl::conv2d_wg<half_t>(a, ns, "pulp_conv2d_fp16_bw_param_grads_cl");
}
int ptl_conv2d_fp16_ig_batched(const struct Conv2D_args_fp16 *a, int ns) {
    return ptl::conv2d_ig<half_t>(a, ns, "pulp_conv2d_fp16_bw_input_grads_cl");
}
int ptl_conv2d_fp32_bw_batched(const struct Conv2D_args *a, int ns) {
    return ptl::conv2d_bw<float>(a, ns, "pulp_conv2d_fp32_bw_cl");
}
int ptl_conv2d_fp16_bw_batched(const struct Conv2D_args_fp16 *a, int ns) {
    return ptl::conv2d_bw<half_t>(a, ns, "pulp_conv2d_fp16_bw_cl");
}

size_t ptl_conv2d_fp16_cache_bytes(const struct Conv2D_args_fp16 *a, int ns) {
    ptl::ConvGeom g;
    if (ns <= 0 || ptl::conv_geom(a, g, "ptl_conv2d_fp16_cache_bytes", false)) return 0;
    if (g.hwc || g.Hk != 3 || g.Wk != 3 || g.sh != 1 || g.sw != 1 || g.Ci % 64 != 0) return 0;
    ptl::ConvTileDesc d = {};
    d.batch = ns; d.Cin = g.Ci; d.Hin = g.H; d.Win = g.W;
    d.Cout = g.Co; d.Ho = g.Ho; d.Wo = g.Wo;
    d.KH = 3; d.KW = 3; d.sh = 1; d.sw = 1;
    d.padU = g.Up; d.padD = g.Dp; d.padL = g.Lp; d.padR = g.Rp;
    int Hp, Wp;
    ptl::conv_padded_grid(d, &Hp, &Wp);
    if (!ptl::conv_halo_fits(d, Hp, Wp)) return 0;
    return ((size_t)(g.Ci / 8) * ns * Hp * Wp + (size_t)ptl::conv_halo_margin()) * 16;
}
int ptl_conv2d_fp16_fw_batched_cached(const struct Conv2D_args_fp16 *a, int ns, struct ptl_conv_cache *c) {
    if (c) c->valid = 0;
    ptl::conv_cache_set(c, nullptr);
    const int rc = ptl::conv2d_fw<half_t>(a, ns, "pulp_conv2d_fp16_fw_cl");
    ptl::conv_cache_set(nullptr, nullptr);
    return rc;
}
int ptl_conv2d_fp16_cache_prepare(const struct Conv2D_args_fp16 *reader, int ns, struct ptl_conv_cache *c) {
    if (!c) {
        ptl::set_error("ptl_conv2d_fp16_cache_prepare: no cache");
        return 1;
    }
    c->valid = 0;
    const size_t need = ptl_conv2d_fp16_cache_bytes(reader, ns);
    ptl::ConvGeom g;
    if (need == 0 || ptl::conv_geom(reader, g, "ptl_conv2d_fp16_cache_prepare", false)) {
        ptl::set_error("ptl_conv2d_fp16_cache_prepare: the layer does not read a blocked copy of its input");
        return 1;
    }
    if (!c->buf || c->bytes < need || reinterpret_cast<uintptr_t>(c->buf) % 16 != 0) {
        ptl::set_error("ptl_conv2d_fp16_cache_prepare: the buffer must be 16-byte aligned device memory of %zu bytes", need);
        return 1;
    }
    if (!ptl::ensure_init()) return 2;
    // zero halo, zero margin: the producing layer only ever writes the pixels
    const size_t n = need / 2;  // halves, 8 per thread
    hipLaunchKernelGGL((ptl::zero_kernel<half_t>), dim3(ptl::blocks_for((n + 7) / 8)), dim3(256), 0, ptl::state().stream,
                       static_cast<half_t *>(c->buf), n, 8);
    if (!ptl::hip_ok(hipGetLastError(), "zero launch")) return 2;
    ptl::ConvTileDesc d = {};
    d.Hin = g.H; d.Win = g.W; d.padU = g.Up; d.padD = g.Dp; d.padL = g.Lp; d.padR = g.Rp;
    int Hp, Wp;
    ptl::conv_padded_grid(d, &Hp, &Wp);
    const int geo[6] = {ns, g.Ci, Hp, Wp, g.Up, g.Lp};
    for (int i = 0; i < 6; ++i) c->geometry[i] = geo[i];
    return 0;
}
int ptl_conv2d_fp16_fw_batched_chained(const struct Conv2D_args_fp16 *a, int ns, struct ptl_conv_cache *in,
                                       struct ptl_conv_cache *out) {
    if (out) out->valid = 0;
    // (a bias is added by a launch behind the convolution kernel: the copy would miss it, so none is written)
    if (a && a->USE_BIASES == 1) out = nullptr;
    const bool have = in && in->valid;
    ptl::conv_cache_set(have ? nullptr : in, nullptr);
    ptl::conv_cache_chain(have ? in : nullptr, out);
    const int rc = ptl::conv2d_fw<half_t>(a, ns, "pulp_conv2d_fp16_fw_cl");
    ptl::conv_cache_set(nullptr, nullptr);
    ptl::conv_cache_chain(nullptr, nullptr);
    return rc;
}
int ptl_conv2d_fp16_wg_batched_cached(const struct Conv2D_args_fp16 *a, int ns, const struct ptl_conv_cache *c) {
    ptl::conv_cache_set(nullptr, c);
    const int rc = ptl::conv2d_wg<half_t>(a, ns, "pulp_conv2d_fp16_bw_param_grads_cl");
    ptl::conv_cache_set(nullptr, nullptr);
    return rc;
}
int ptl_conv2d_fp16_bw_batched_cached(const struct Conv2D_args_fp16 *a, int ns, const struct ptl_conv_cache *c) {
    ptl::conv_cache_set(nullptr, c);
    const int rc = ptl::conv2d_bw<half_t>(a, ns, "pulp_conv2d_fp16_bw_cl");
    ptl::conv_cache_set(nullptr, nullptr);
    return rc;
}

int ptl_conv2d_fp16_bw_batched_deferred(const struct Conv2D_args_fp16 *a, int ns, struct ptl_wg_batch *batch) {
    ptl::conv_small_defer_to(batch);
    const int rc = ptl::conv2d_bw<half_t>(a, ns, "pulp_conv2d_fp16_bw_cl");
    ptl::conv_small_defer_to(nullptr);
    return rc;
}
int ptl_conv2d_fp32_bw_batched_deferred(const struct Conv2D_args *a, int ns, struct ptl_wg_batch *batch) {
    ptl::conv_small_defer_to(batch);
    const int rc = ptl::conv2d_bw<float>(a, ns, "pulp_conv2d_fp32_bw_cl");
    ptl::conv_small_defer_to(nullptr);
    return rc;
}
int ptl_conv2d_fp16_fw_batched_normed(const struct Conv2D_args_fp16 *a, int ns, struct ptl_norm_stats *st,
                                      const struct BatchNorm_args_fp16 *norm, const struct ptl_norm_fusion_fp16 *f,
                                      const struct ptl_norm_stats *norm_st) {
    return ptl::conv2d_fw_normed<half_t>(a, ns, st, norm, f, norm_st, ptl_batch_norm_fused_fp16_fw_stats,
                                         "pulp_conv2d_fp16_fw_cl");
}
int ptl_conv2d_fp32_fw_batched_normed(const struct Conv2D_args *a, int ns, struct ptl_norm_stats *st,
                                      const struct BatchNorm_args_fp32 *norm, const struct ptl_norm_fusion_fp32 *f,
                                      const struct ptl_norm_stats *norm_st) {
    return ptl::conv2d_fw_normed<float>(a, ns, st, norm, f, norm_st, ptl_batch_norm_fused_fp32_fw_stats,
                                        "pulp_conv2d_fp32_fw_cl");
}
int ptl_conv2d_fp16_bw_batched_deferred_post(const struct Conv2D_args_fp16 *a, int ns, struct ptl_wg_batch *batch,
                                             const struct ptl_grad_post *post, struct ptl_norm_stats *sums) {
    return ptl::conv2d_bw_post<half_t>(a, ns, batch, post, sums, "pulp_conv2d_fp16_bw_cl");
}
int ptl_conv2d_fp32_bw_batched_deferred_post(const struct Conv2D_args *a, int ns, struct ptl_wg_batch *batch,
                                             const struct ptl_grad_post *post, struct ptl_norm_stats *sums) {
    return ptl::conv2d_bw_post<float>(a, ns, batch, post, sums, "pulp_conv2d_fp32_bw_cl");
}
int ptl_conv2d_fp16_fw_batched_stats(const struct Conv2D_args_fp16 *a, int ns, struct ptl_norm_stats *st) {
    return ptl::conv2d_fw_stats<half_t>(a, ns, st, "pulp_conv2d_fp16_fw_cl");
}
int ptl_conv2d_fp32_fw_batched_stats(const struct Conv2D_args *a, int ns, struct ptl_norm_stats *st) {
    return ptl::conv2d_fw_stats<float>(a, ns, st, "pulp_conv2d_fp32_fw_cl");
}
int ptl_conv2d_fp16_wg_flush(struct ptl_wg_batch *batch) { return ptl::conv_small_flush<half_t>(batch); }
int ptl_conv2d_fp32_wg_flush(struct ptl_wg_batch *batch) { return ptl::conv_small_flush<float>(batch); }

int ptl_conv_pw_fp32_fw_batched(const struct PointWise_Conv_args *a, int ns) {
    return ptl::pw_step<float>(a, ns, STEP_FW, "pulp_conv_pw_fp32_fw_cl");
}
int ptl_conv_pw_fp32_wg_batched(const struct PointWise_Conv_args *a, int ns) {
    return ptl::pw_step<float>(a, ns, STEP_WGT_GRAD, "pulp_conv_pw_fp32_bw_param_grads_cl");
}
int ptl_conv_pw_fp32_ig_batched(const struct PointWise_Conv_args *a, int ns) {
    return ptl::pw_step<float>(a, ns, STEP_IN_GRAD, "pulp_conv_pw_fp32_bw_input_grads_cl");
}
int ptl_conv_pw_fp16_fw_batched(const struct PointWise_Conv_args_fp16 *a, int ns) {
    return ptl::pw_step<half_t>(a, ns, STEP_FW, "pulp_conv_pw_fp16_fw_cl");
}
int ptl_conv_pw_fp16_wg_batched(const struct PointWise_Conv_args_fp16 *a, int ns) {
    return ptl::pw_step<half_t>(a, ns, STEP_WGT_GRAD, "pulp_conv_pw_fp16_bw_param_grads_cl");
}
int ptl_conv_pw_fp16_ig_batched(const struct PointWise_Conv_args_fp16 *a, int ns) {
    return ptl::pw_step<half_t>(a, ns, STEP_IN_GRAD, "pulp_conv_pw_fp16_bw_input_grads_cl");
}

int ptl_linear_fp32_fw_batched(const struct Linear_args *a, int ns) {
    return ptl::linear_step<float>(a, ns, STEP_FW, "pulp_linear_fp32_fw_cl");
}
int ptl_linear_fp32_wg_batched(const struct Linear_args *a, int ns) {
    return ptl::linear_step<float>(a, ns, STEP_WGT_GRAD, "pulp_linear_fp32_bw_param_grads_cl");
}
int ptl_linear_fp32_ig_batched(const struct Linear_args *a, int ns) {
    return ptl::linear_step<float>(a, ns, STEP_IN_GRAD, "pulp_linear_fp32_bw_input_grads_cl");
}
int ptl_linear_fp16_fw_batched(const struct Linear_args_fp16 *a, int ns) {
    return ptl::linear_step<half_t>(a, ns, STEP_FW, "pulp_linear_fp16_fw_cl");
}
int ptl_linear_fp16_wg_batched(const struct Linear_args_fp16 *a, int ns) {
    return ptl::linear_step<half_t>(a, ns, STEP_WGT_GRAD, "pulp_linear_fp16_bw_param_grads_cl");
}
int ptl_linear_fp32_bw_batched(const struct Linear_args *a, int ns) {
    if (a && (a->skip_wg_grad || a->skip_in_grad || ns == 1)) {  // one of the two, or one sample: the single steps
        int rc = a->skip_wg_grad ? 0 : ptl::linear_step<float>(a, ns, STEP_WGT_GRAD, "pulp_linear_fp32_bw_cl");
        if (rc == 0 && !a->skip_in_grad) rc = ptl::linear_step<float>(a, ns, STEP_IN_GRAD, "pulp_linear_fp32_bw_cl");
        return rc;
    }
    if (ns == 1) {
        int rc = ptl::linear_step<float>(a, 1, STEP_WGT_GRAD, "pulp_linear_fp32_bw_cl");
        return rc ? rc : ptl::linear_step<float>(a, 1, STEP_IN_GRAD, "pulp_linear_fp32_bw_cl");
    }
    return ptl::linear_step<float>(a, ns, STEP_BW_BOTH, "pulp_linear_fp32_bw_cl");
}
int ptl_linear_fp16_bw_batched(const struct Linear_args_fp16 *a, int ns) {
    if (a && (a->skip_wg_grad || a->skip_in_grad || ns == 1)) {  // one of the two, or one sample: the single steps
        int rc = a->skip_wg_grad ? 0 : ptl::linear_step<half_t>(a, ns, STEP_WGT_GRAD, "pulp_linear_fp16_bw_cl");
        if (rc == 0 && !a->skip_in_grad) rc = ptl::linear_step<half_t>(a, ns, STEP_IN_GRAD, "pulp_linear_fp16_bw_cl");
        return rc;
    }
    if (ns == 1) {
        int rc = ptl::linear_step<half_t>(a, 1, STEP_WGT_GRAD, "pulp_linear_fp16_bw_cl");
        return rc ? rc : ptl::linear_step<half_t>(a, 1, STEP_IN_GRAD, "pulp_linear_fp16_bw_cl");
    }
    return ptl::linear_step<half_t>(a, ns, STEP_BW_BOTH, "pulp_linear_fp16_bw_cl");
}
int ptl_linear_fp16_ig_batched(const struct Linear_args_fp16 *a, int ns) {
    return ptl::linear_step<half_t>(a, ns, STEP_IN_GRAD, "pulp_linear_fp16_bw_input_grads_cl");
}

int ptl_mm_fp32(const float *A, const float *B, float *C, int N, int M, int K, int trans_B) {
    if (N < 0 || M < 0 || K < 0 || !A || !B || !C) {
        ptl::set_error("ptl_mm_fp32: invalid arguments");
        return 1;
    }
    if (!ptl::ensure_init()) return 2;
    ptl::Stager sg;
    const float *dA = sg.in(A, (size_t)N * K);
    const float *dB = sg.in(B, (size_t)K * M);
    float *dC = K > 0 ? sg.out(C, (size_t)N * M) : C;
    if (sg.failed()) return 2;
    return sg.finish(ptl::mm_dispatch<float>(dA, dB, dC, N, M, K, trans_B));
}

int ptl_mm_fp16(const fp16 *A, const fp16 *B, fp16 *C, int N, int M, int K, int trans_B) {
    if (N < 0 || M < 0 || K < 0 || !A || !B || !C) {
        ptl::set_error("ptl_mm_fp16: invalid arguments");
        return 1;
    }
    if (!ptl::ensure_init()) return 2;
    ptl::Stager sg;
    const half_t *dA = sg.in(reinterpret_cast<const half_t *>(A), (size_t)N * K);
    const half_t *dB = sg.in(reinterpret_cast<const half_t *>(B), (size_t)K * M);
    half_t *dC = K > 0 ? sg.out(reinterpret_cast<half_t *>(C), (size_t)N * M) : reinterpret_cast<half_t *>(C);
    if (sg.failed()) return 2;
    return sg.finish(ptl::mm_dispatch<half_t>(dA, dB, dC, N, M, K, trans_B));
}

}  // extern "C"
