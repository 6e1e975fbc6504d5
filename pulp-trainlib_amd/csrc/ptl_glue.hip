// Layers around the matmul core in a ResNet-style training step: ReLU, residual connection, average
// pooling, cross-entropy loss, gradient descent, batch normalisation (forward).  All are bandwidth-bound
// element or small-reduction kernels; fp16 tensors are read as IEEE half, computed in fp32 and rounded once.
#include <float.h>
#include <type_traits>

#include "ptl_api.h"
#include "ptl_conv_tile.hpp"
#include "ptl_host.hpp"
#include "ptl_norm_fold.hpp"
#include "ptl_structs.h"

namespace ptl {

static inline unsigned glue_blocks(size_t n) { return (unsigned)((n + 255) / 256); }

static int glue_bad(const char *fn, const char *what) {
    printf("[%s] %s\n", fn, what);
    set_error("%s: %s", fn, what);
    return 1;
}

// ---- ReLU (lib/sources/pulp_act_fp32.c:95-129) ------------------------------------------------------
// Element-wise maps c = op(a, b) on 16-byte vectors (tensors that are 16-byte aligned; the last n % VEC elements
// go one by one).  The one-element-per-thread kernels below remain for unaligned tensors.
struct OpReluFw {
    __device__ static float map(float a, float) { return a > 0.f ? a : 0.f; }
};
struct OpReluBw {
    __device__ static float map(float x, float dy) { return x > 0.f ? dy : 0.f; }
};
struct OpAdd {
    __device__ static float map(float a, float b) { return a + b; }
};
struct OpCopy {
    __device__ static float map(float a, float) { return a; }
};

template <typename T, typename Op, bool TWO>
__global__ __launch_bounds__(256) void ew_vec_kernel(const T *a, const T *b, T *c, size_t n) {  // c may be a or b
    constexpr int VEC = 16 / (int)sizeof(T);
    union V {
        uint4 raw;
        T e[VEC];
    };
    const size_t nvec = n / VEC, v = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (v < nvec) {
        V x, y;
        x.raw = reinterpret_cast<const uint4 *>(a)[v];
        if (TWO) y.raw = reinterpret_cast<const uint4 *>(b)[v];
#pragma unroll
        for (int q = 0; q < VEC; ++q) x.e[q] = (T)Op::map((float)x.e[q], TWO ? (float)y.e[q] : 0.f);
        reinterpret_cast<uint4 *>(c)[v] = x.raw;
    }
    if (blockIdx.x == 0) {
        const size_t i = nvec * VEC + threadIdx.x;
        if (i < n) c[i] = (T)Op::map((float)a[i], TWO ? (float)b[i] : 0.f);
    }
}

// Launches the vector form when the tensors allow it; false = the caller launches its element kernel.
template <typename T, typename Op, bool TWO>
static bool ew_vec_launch(const T *a, const T *b, T *c, size_t n) {
    constexpr int VEC = 16 / (int)sizeof(T);
    auto al = [](const void *p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; };
    if (n < (size_t)VEC || !al(a) || !al(c) || (TWO && !al(b))) return false;
    hipLaunchKernelGGL((ew_vec_kernel<T, Op, TWO>), dim3(glue_blocks((n / VEC))), dim3(256), 0, state().stream, a, b, c,
                       n);
    return true;
}

template <typename T>
__global__ __launch_bounds__(256) void relu_fw_kernel(const T *__restrict__ x, T *__restrict__ y, size_t n) {
    size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) y[i] = (float)x[i] > 0.f ? x[i] : (T)0.f;
}

template <typename T>
__global__ __launch_bounds__(256) void relu_bw_kernel(const T *__restrict__ x, const T *__restrict__ dy,
                                                      T *__restrict__ dx, size_t n) {
    size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) dx[i] = (float)x[i] > 0.f ? dy[i] : (T)0.f;
}

template <typename T, typename Args>
static int relu_step(const Args *a, int ns, int step, const char *fn) {
    if (!a || !a->input || !a->output || a->input->dim <= 0) return glue_bad(fn, "invalid arguments");
    if (ns <= 0) return 0;
    if (!ensure_init()) return 2;
    const size_t n = (size_t)ns * a->input->dim;
    Stager sg;
    const T *x = sg.in(reinterpret_cast<const T *>(a->input->data), n);
    if (step == 0) {
        T *y = sg.out(reinterpret_cast<T *>(a->output->data), n);
        if (sg.failed() || !x || !y) return sg.failed() ? 2 : glue_bad(fn, "null buffer");
        if (!ew_vec_launch<T, OpReluFw, false>(x, (const T *)nullptr, y, n))
            hipLaunchKernelGGL((relu_fw_kernel<T>), dim3(glue_blocks(n)), dim3(256), 0, state().stream, x, y, n);
    } else {
        const T *dy = sg.in(reinterpret_cast<const T *>(a->output->diff), n);
        T *dx = sg.out(reinterpret_cast<T *>(a->input->diff), n);
        if (sg.failed() || !x || !dy || !dx) return sg.failed() ? 2 : glue_bad(fn, "null buffer");
        if (!ew_vec_launch<T, OpReluBw, true>(x, dy, dx, n))
            hipLaunchKernelGGL((relu_bw_kernel<T>), dim3(glue_blocks(n)), dim3(256), 0, state().stream, x, dy, dx, n);
    }
    return sg.finish(hip_ok(hipGetLastError(), "relu launch") ? 0 : 2);
}

// ---- Residual connection (lib/sources/pulp_residual_fp32.c:26-113) ----------------------------------
template <typename T>
__global__ __launch_bounds__(256) void add_kernel(const T *__restrict__ a, const T *__restrict__ b, T *__restrict__ c,
                                                  size_t n) {
    size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) c[i] = (T)((float)a[i] + (float)b[i]);
}

template <typename T>
__global__ __launch_bounds__(256) void copy_elems_kernel(const T *__restrict__ a, T *__restrict__ c, size_t n) {
    size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) c[i] = a[i];
}

template <typename T, typename Args>
static int residual_step(const Args *a, int ns, int step, const char *fn) {
    if (!a || !a->skip || !a->lout || !a->output) return glue_bad(fn, "invalid arguments");
    const int dim = a->output->dim;
    if (step == 0 && (a->skip->dim != a->lout->dim || a->lout->dim != dim))
        return glue_bad(fn, "Sizes of input and output activations not matching!!");
    if (step == 1 && a->skip_in_grad == 0 && a->skip->dim != dim)
        return glue_bad(fn, "Sizes of input and output activations not matching!!");
    if (step == 2 && a->lout->dim != dim) return glue_bad(fn, "Sizes of input and output activations not matching!!");
    if (ns <= 0 || dim <= 0) return 0;
    if (step == 1 && a->skip_in_grad != 0) return 0;
    if (!ensure_init()) return 2;
    const size_t n = (size_t)ns * dim;
    Stager sg;
    if (step == 0) {
        const T *s = sg.in(reinterpret_cast<const T *>(a->skip->data), n);
        const T *l = sg.in(reinterpret_cast<const T *>(a->lout->data), n);
        T *o = sg.out(reinterpret_cast<T *>(a->output->data), n);
        if (sg.failed() || !s || !l || !o) return sg.failed() ? 2 : glue_bad(fn, "null buffer");
        if (!ew_vec_launch<T, OpAdd, true>(s, l, o, n))
            hipLaunchKernelGGL((add_kernel<T>), dim3(glue_blocks(n)), dim3(256), 0, state().stream, s, l, o, n);
    } else if (step == 1) {
        const T *g = sg.in(reinterpret_cast<const T *>(a->output->diff), n);
        T *s = sg.inout(reinterpret_cast<T *>(a->skip->diff), n);
        if (sg.failed() || !g || !s) return sg.failed() ? 2 : glue_bad(fn, "null buffer");
        if (!ew_vec_launch<T, OpAdd, true>(g, (const T *)s, s, n))
            hipLaunchKernelGGL((add_kernel<T>), dim3(glue_blocks(n)), dim3(256), 0, state().stream, g, s, s, n);
    } else {
        const T *g = sg.in(reinterpret_cast<const T *>(a->output->diff), n);
        T *l = sg.out(reinterpret_cast<T *>(a->lout->diff), n);
        if (sg.failed() || !g || !l) return sg.failed() ? 2 : glue_bad(fn, "null buffer");
        if (!ew_vec_launch<T, OpCopy, false>(g, (const T *)nullptr, l, n))
            hipLaunchKernelGGL((copy_elems_kernel<T>), dim3(glue_blocks(n)), dim3(256), 0, state().stream, g, l, n);
    }
    return sg.finish(hip_ok(hipGetLastError(), "residual launch") ? 0 : 2);
}

// ---- Average pooling (lib/sources/pulp_pooling_fp32.c:24-122) ---------------------------------------
struct PoolGeom {
    int C, H, W, Ho, Wo, Hk, Wk, Hs, Ws, Hact, Wact;
};

// One wave per output element: lanes stride over the window.
template <typename T>
__global__ __launch_bounds__(256) void avgpool_fw_kernel(const T *__restrict__ x, T *__restrict__ y, PoolGeom g,
                                                         size_t nout) {
    const size_t o = (size_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    if (o >= nout) return;
    const int wa = (int)(o % g.Wact), ha = (int)((o / g.Wact) % g.Hact);
    const size_t plane = o / ((size_t)g.Wact * g.Hact);  // sample * C + channel
    const T *src = x + plane * g.H * g.W;
    float s = 0.f;
    for (int e = lane; e < g.Hk * g.Wk; e += 64) {
        const int hk = e / g.Wk, wk = e - hk * g.Wk;
        s += (float)src[(size_t)(ha * g.Hs + hk) * g.W + wa * g.Ws + wk];
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) s += __shfl_xor(s, off);
    if (lane == 0) y[plane * g.Ho * g.Wo + (size_t)ha * g.Wo + wa] = (T)(s / (float)(g.Hk * g.Wk));
}

// One thread per input element: sums the output gradients of the windows that contain it.
template <typename T>
__global__ __launch_bounds__(256) void avgpool_bw_kernel(const T *__restrict__ dy, T *__restrict__ dx, PoolGeom g,
                                                         size_t nin) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= nin) return;
    const int w = (int)(i % g.W), h = (int)((i / g.W) % g.H);
    const size_t plane = i / ((size_t)g.W * g.H);
    const T *src = dy + plane * g.Ho * g.Wo;
    float s = 0.f;
    for (int ho = 0; ho < g.Ho; ++ho) {
        const int hk = h - ho * g.Hs;
        if (hk < 0 || hk >= g.Hk) continue;
        for (int wo = 0; wo < g.Wo; ++wo) {
            const int wk = w - wo * g.Ws;
            if (wk < 0 || wk >= g.Wk) continue;
            s += (float)src[(size_t)ho * g.Wo + wo] / (float)(g.Hk * g.Wk);
        }
    }
    dx[i] = (T)s;
}

template <typename T, typename Args>
static int avgpool_step(const Args *a, int ns, int step, const char *fn) {
    if (!a || !a->input || !a->output) return glue_bad(fn, "invalid arguments");
    PoolGeom g;
    g.C = a->input->C;
    g.H = a->input->H;
    g.W = a->input->W;
    g.Ho = a->output->H;
    g.Wo = a->output->W;
    g.Hk = a->Hker;
    g.Wk = a->Wker;
    g.Hs = a->Hstride;
    g.Ws = a->Wstride;
    if (g.C <= 0 || g.H <= 0 || g.W <= 0 || g.Hk <= 0 || g.Wk <= 0 || g.Hs <= 0 || g.Ws <= 0 || g.Hk > g.H ||
        g.Wk > g.W)
        return glue_bad(fn, "invalid pooling geometry");
    g.Hact = (g.H - g.Hk + g.Hs) / g.Hs;
    g.Wact = (g.W - g.Wk + g.Ws) / g.Ws;
    if (g.Hact != g.Ho || g.Wact != g.Wo) return glue_bad(fn, "Invalid pooling kernel size or output size!");
    if (ns <= 0) return 0;
    if (!ensure_init()) return 2;
    const size_t nin = (size_t)ns * g.C * g.H * g.W, nout = (size_t)ns * g.C * g.Ho * g.Wo;
    Stager sg;
    if (step == 0) {
        const T *x = sg.in(reinterpret_cast<const T *>(a->input->data), nin);
        T *y = sg.out(reinterpret_cast<T *>(a->output->data), nout);
        if (sg.failed() || !x || !y) return sg.failed() ? 2 : glue_bad(fn, "null buffer");
        hipLaunchKernelGGL((avgpool_fw_kernel<T>), dim3((unsigned)((nout + 3) / 4)), dim3(256), 0, state().stream, x,
                           y, g, nout);
    } else {
        const T *dy = sg.in(reinterpret_cast<const T *>(a->output->diff), nout);
        T *dx = sg.out(reinterpret_cast<T *>(a->input->diff), nin);
        if (sg.failed() || !dy || !dx) return sg.failed() ? 2 : glue_bad(fn, "null buffer");
        hipLaunchKernelGGL((avgpool_bw_kernel<T>), dim3(glue_blocks(nin)), dim3(256), 0, state().stream, dy, dx, g,
                           nin);
    }
    return sg.finish(hip_ok(hipGetLastError(), "pooling launch") ? 0 : 2);
}

// ---- Cross-entropy over raw logits (lib/sources/pulp_losses_fp32.c:26-138) ---------------------------
// One wave per sample; lanes stride over the classes.
template <typename T>
__global__ __launch_bounds__(256) void cross_entropy_kernel(const T *__restrict__ logits, const T *__restrict__ target,
                                                            T *__restrict__ loss, T *__restrict__ grad, int ncls,
                                                            int ns, int backward) {
    const int b = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (b >= ns) return;
    const T *z = logits + (size_t)b * ncls, *y = target + (size_t)b * ncls;
    float mx = -FLT_MAX;
    for (int i = lane; i < ncls; i += 64) mx = fmaxf(mx, (float)z[i]);
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off));
    float se = 0.f, dot = 0.f, sy = 0.f;
    for (int i = lane; i < ncls; i += 64) {
        se += expf((float)z[i] - mx);
        dot += (float)y[i] * (float)z[i];
        sy += (float)y[i];
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        se += __shfl_xor(se, off);
        dot += __shfl_xor(dot, off);
        sy += __shfl_xor(sy, off);
    }
    if (!backward) {
        if (sizeof(T) == 4 && sy == 0.f) sy = 1.0f;  // only the fp32 forward guards this (pulp_losses_fp32.c:66-69)
        if (lane == 0) loss[b] = (T)(-(dot - (logf(se) + mx) * sy));
    } else {
        if (sy == 0.f) sy = 1.0f;
        const float inv = 1.0f / se;
        for (int i = lane; i < ncls; i += 64)
            grad[(size_t)b * ncls + i] = (T)((expf((float)z[i] - mx) * inv) * sy - (float)y[i]);
    }
}

template <typename T, typename Args>
static int cross_entropy_step(const Args *a, int ns, int step, const char *fn) {
    if (!a || !a->output || !a->target || a->output->dim <= 0) return glue_bad(fn, "invalid arguments");
    if (ns <= 0) return 0;
    if (!ensure_init()) return 2;
    const int ncls = a->output->dim;
    const size_t n = (size_t)ns * ncls;
    Stager sg;
    const T *z = sg.in(reinterpret_cast<const T *>(a->output->data), n);
    const T *y = sg.in(reinterpret_cast<const T *>(a->target), n);
    T *loss = nullptr, *grad = nullptr;
    if (step == 0)
        loss = sg.out(reinterpret_cast<T *>(a->wr_loss), (size_t)ns);
    else
        grad = sg.out(reinterpret_cast<T *>(a->output->diff), n);
    if (sg.failed() || !z || !y || (step == 0 ? !loss : !grad)) return sg.failed() ? 2 : glue_bad(fn, "null buffer");
    hipLaunchKernelGGL((cross_entropy_kernel<T>), dim3((ns + 3) / 4), dim3(256), 0, state().stream, z, y, loss, grad,
                       ncls, ns, step);
    return sg.finish(hip_ok(hipGetLastError(), "loss launch") ? 0 : 2);
}

// ---- Global average pooling, classifier and loss of a batch, forward and backward, in one launch ----------------
// What six calls do one after the other on tensors of a few hundred elements per sample (pooling forward, Linear
// forward, cross-entropy forward and backward, Linear backward, pooling backward: 31 us of launches for a ResNet-20 at
// batch 128): a workgroup per sample keeps the sample's pooled vector, logits and gradients in LDS and writes every
// tensor the six calls write, rounded to the tensor type where they round.  The pooling and the loss repeat the
// arithmetic of their kernels above; the classifier's dot products are added up lane-strided and by a butterfly, not
// in the order of the MFMA product, so logits and what follows agree with the six calls to rounding.  The weight
// gradient is a sum over the samples: every workgroup leaves its sample's outer product as a part of a deferred batch
// (in the order wg_small_flush_kernel reads), and the flush adds them up.
struct HeadArgs {
    const void *x, *w, *target;
    void *pooled, *logits, *loss, *dlogits, *dpooled, *dx;
    float *part;  // [sample][32-channel block][class][channel of the block]
    int C, HW, ncls, cbi_n, cols_kept;
};

template <typename T>
__global__ __launch_bounds__(256) void head_kernel(const HeadArgs a) {
    extern __shared__ float head_lds[];
    float *pooled = head_lds, *dpool = pooled + a.C, *logit = dpool + a.C, *dlog = logit + a.ncls;
    float *Wl = dlog + a.ncls, *yl = Wl + a.ncls * a.C;  // the classifier's weights and the sample's target
    const int n = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const T *x = reinterpret_cast<const T *>(a.x) + (size_t)n * a.C * a.HW;
    // (everything the later phases read from memory is asked for now, with the planes' loads)
    for (int i = tid; i < a.ncls * a.C; i += 256) Wl[i] = (float)reinterpret_cast<const T *>(a.w)[i];
    for (int i = tid; i < a.ncls; i += 256) yl[i] = (float)reinterpret_cast<const T *>(a.target)[(size_t)n * a.ncls + i];
    // pooling forward: a wave per channel, lanes stride over the plane (avgpool_fw_kernel's order), eight channels of
    // a wave at a time so that their loads are in the air together and their butterflies side by side
    for (int c0 = wave; c0 < a.C; c0 += 32) {
        float s[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int c = c0 + 4 * u;
            s[u] = 0.f;
            if (c < a.C)
                for (int e = lane; e < a.HW; e += 64) s[u] += (float)x[(size_t)c * a.HW + e];
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1)
#pragma unroll
            for (int u = 0; u < 8; ++u) s[u] += __shfl_xor(s[u], off);
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int c = c0 + 4 * u;
            if (lane == 0 && c < a.C) {
                const T p = (T)(s[u] / (float)a.HW);
                reinterpret_cast<T *>(a.pooled)[(size_t)n * a.C + c] = p;
                pooled[c] = (float)p;
            }
        }
    }
    __syncthreads();
    // classifier forward: a wave per class, the (at most eight) classes of a wave side by side
    {
        float s[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int k = wave + 4 * u;
            s[u] = 0.f;
            if (k < a.ncls)
                for (int c = lane; c < a.C; c += 64) s[u] += pooled[c] * Wl[k * a.C + c];
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1)
#pragma unroll
            for (int u = 0; u < 8; ++u) s[u] += __shfl_xor(s[u], off);
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int k = wave + 4 * u;
            if (lane == 0 && k < a.ncls) {
                const T z = (T)s[u];
                reinterpret_cast<T *>(a.logits)[(size_t)n * a.ncls + k] = z;
                logit[k] = (float)z;
            }
        }
    }
    __syncthreads();
    // loss and its gradient: the first wave (cross_entropy_kernel's arithmetic, both passes)
    if (wave == 0) {
        const float *y = yl;
        float mx = -FLT_MAX;
        for (int i = lane; i < a.ncls; i += 64) mx = fmaxf(mx, logit[i]);
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off));
        float se = 0.f, dot = 0.f, sy = 0.f;
        for (int i = lane; i < a.ncls; i += 64) {
            se += expf(logit[i] - mx);
            dot += y[i] * logit[i];
            sy += y[i];
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            se += __shfl_xor(se, off);
            dot += __shfl_xor(dot, off);
            sy += __shfl_xor(sy, off);
        }
        float sy_fw = sy;
        if (sizeof(T) == 4 && sy_fw == 0.f) sy_fw = 1.0f;  // (only the fp32 forward guards this)
        if (lane == 0) reinterpret_cast<T *>(a.loss)[n] = (T)(-(dot - (logf(se) + mx) * sy_fw));
        if (sy == 0.f) sy = 1.0f;
        const float inv = 1.0f / se;
        for (int i = lane; i < a.ncls; i += 64) {
            const T g = (T)((expf(logit[i] - mx) * inv) * sy - y[i]);
            reinterpret_cast<T *>(a.dlogits)[(size_t)n * a.ncls + i] = g;
            dlog[i] = (float)g;
        }
    }
    __syncthreads();
    // classifier backward: the gradient of the pooled vector, and this sample's part of the weight gradient
    for (int c = tid; c < a.C; c += 256) {
        float s = 0.f;
        for (int k = 0; k < a.ncls; ++k) s += dlog[k] * Wl[k * a.C + c];
        const T g = (T)s;
        reinterpret_cast<T *>(a.dpooled)[(size_t)n * a.C + c] = g;
        dpool[c] = (float)g;
    }
    float *part = a.part + (size_t)n * a.cbi_n * a.ncls * a.cols_kept;
    for (int i = tid; i < a.cbi_n * a.ncls * a.cols_kept; i += 256) {
        const int col = i % a.cols_kept, k = (i / a.cols_kept) % a.ncls, cbi = i / (a.cols_kept * a.ncls);
        const int c = cbi * 32 + col;
        part[i] = c < a.C ? dlog[k] * pooled[c] : 0.f;
    }
    __syncthreads();
    // pooling backward: every element of a plane gets its channel's share (avgpool_bw_kernel with one window)
    T *dx = reinterpret_cast<T *>(a.dx) + (size_t)n * a.C * a.HW;
    constexpr int VEC = 16 / (int)sizeof(T);
    if (a.HW % VEC == 0 && (reinterpret_cast<uintptr_t>(a.dx) % 16) == 0) {  // (planes of whole 16-byte pieces)
        const int pieces = a.HW / VEC;
        for (int i = tid; i < a.C * pieces; i += 256) {
            const T v = (T)(dpool[i / pieces] / (float)a.HW);
            union {
                uint4 raw;
                T e[VEC];
            } o;
#pragma unroll
            for (int j = 0; j < VEC; ++j) o.e[j] = v;
            reinterpret_cast<uint4 *>(dx)[i] = o.raw;
        }
    } else {
        for (int i = tid; i < a.C * a.HW; i += 256) dx[i] = (T)(dpool[i / a.HW] / (float)a.HW);
    }
}

template <typename T, typename Pool, typename Lin, typename Loss>
static int head_step(const Pool *pa, const Lin *la, const Loss *ca, int ns, ::ptl_wg_batch *batch,
                     int (*pool_call)(const Pool *, int, int), int (*lin_fw)(const Lin *, int),
                     int (*lin_bw)(const Lin *, int), int (*loss_call)(const Loss *, int, int), const char *fn) {
    if (!pa || !la || !ca) return glue_bad(fn, "invalid arguments");
    if (ns <= 0) return 0;
    // one launch: a global pooling whose output is the classifier's input, the classifier's output the loss's, both
    // gradients wanted, no bias, device tensors, room in the batch for the weight gradient's parts
    bool fused = batch && pa->input && pa->output && la->input && la->coeff && la->output && ca->output && ca->target &&
                 ca->wr_loss && pa->Hker == pa->input->H && pa->Wker == pa->input->W && pa->output->H == 1 &&
                 pa->output->W == 1 && pa->input->C > 0 && pa->input->C <= 1024 && pa->input->H * pa->input->W > 0 &&
                 la->input->dim == pa->input->C && la->output->dim > 0 && la->output->dim <= 32 &&
                 (long long)la->output->dim * pa->input->C <= 8192 &&  // (the weights are kept in LDS)
                 ca->output->dim == la->output->dim && la->use_biases != 1 && !la->skip_wg_grad && !la->skip_in_grad &&
                 pa->output->data == la->input->data && pa->output->diff == la->input->diff &&
                 la->output->data == ca->output->data && la->output->diff == ca->output->diff && pa->input->data &&
                 pa->input->diff && pa->output->data && pa->output->diff && la->coeff->data && la->coeff->diff &&
                 la->output->data && la->output->diff && ensure_init();
    if (fused) {
        const int C = pa->input->C, HW = pa->input->H * pa->input->W, ncls = la->output->dim;
        {
            Stager sg(true);  // (host tensors: the six calls, which stage them)
            (void)sg.in(reinterpret_cast<const T *>(pa->input->data), (size_t)ns * C * HW);
            (void)sg.out(reinterpret_cast<T *>(pa->input->diff), (size_t)ns * C * HW);
            (void)sg.out(reinterpret_cast<T *>(pa->output->data), (size_t)ns * C);
            (void)sg.out(reinterpret_cast<T *>(pa->output->diff), (size_t)ns * C);
            (void)sg.in(reinterpret_cast<const T *>(la->coeff->data), (size_t)ncls * C);
            (void)sg.out(reinterpret_cast<T *>(la->coeff->diff), (size_t)ncls * C);
            (void)sg.out(reinterpret_cast<T *>(la->output->data), (size_t)ns * ncls);
            (void)sg.out(reinterpret_cast<T *>(la->output->diff), (size_t)ns * ncls);
            (void)sg.in(reinterpret_cast<const T *>(ca->target), (size_t)ns * ncls);
            (void)sg.out(reinterpret_cast<T *>(ca->wr_loss), (size_t)ns);
            fused = !sg.failed();
        }
        float *part = fused ? wg_batch_reserve(batch, la->coeff->diff, ns, ncls, C, 1) : nullptr;
        if (part) {
            HeadArgs h = {};
            h.x = pa->input->data;
            h.w = la->coeff->data;
            h.target = ca->target;
            h.pooled = pa->output->data;
            h.logits = la->output->data;
            h.loss = ca->wr_loss;
            h.dlogits = la->output->diff;
            h.dpooled = pa->output->diff;
            h.dx = pa->input->diff;
            h.part = part;
            h.C = C;
            h.HW = HW;
            h.ncls = ncls;
            h.cbi_n = (C + 31) / 32;
            h.cols_kept = C < 32 ? C : 32;
            const size_t lds = (size_t)(2 * C + 3 * ncls + ncls * C) * sizeof(float);
            hipLaunchKernelGGL((head_kernel<T>), dim3(ns), dim3(256), lds, state().stream, h);
            return hip_ok(hipGetLastError(), "classifier head launch") ? 0 : 2;
        }
    }
    if (int rc = pool_call(pa, ns, 0)) return rc;
    if (int rc = lin_fw(la, ns)) return rc;
    if (int rc = loss_call(ca, ns, 0)) return rc;
    if (int rc = loss_call(ca, ns, 1)) return rc;
    if (int rc = lin_bw(la, ns)) return rc;
    return pool_call(pa, ns, 1);
}

// ---- Gradient descent (lib/sources/pulp_optimizers_fp32.c:26-104) ------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void sgd_kernel(T *__restrict__ w, T *__restrict__ g, size_t n, float lr,
                                                  float lambda) {
    size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    float gi = (float)g[i], wi = (float)w[i];
    if (lambda != 0.f) {
        gi = gi + lambda * wi;
        g[i] = (T)gi;
        gi = (float)(T)gi;
    }
    w[i] = (T)(wi - lr * gi);
}

template <typename T, typename Args>
static int sgd_step(const Args *a, const char *fn) {
    if (!a || !a->weights) return glue_bad(fn, "invalid arguments");
    if (a->use_biases == 1 && !a->biases) return glue_bad(fn, "use_biases=1 with a null bias blob");
    if (!ensure_init()) return 2;
    const float lr = (float)a->learning_rate, lambda = (float)a->weight_decay_lambda;
    Stager sg;
    const struct { void *data, *diff; int dim; } parts[2] = {
        {a->weights->data, a->weights->diff, a->weights->dim},
        {a->use_biases == 1 ? (void *)a->biases->data : nullptr, a->use_biases == 1 ? (void *)a->biases->diff : nullptr,
         a->use_biases == 1 ? a->biases->dim : 0}};
    for (const auto &p : parts) {
        if (p.dim <= 0) continue;
        if (!p.data || !p.diff) return glue_bad(fn, "null buffer");
        T *w = sg.inout(reinterpret_cast<T *>(p.data), (size_t)p.dim);
        T *g = lambda != 0.f ? sg.inout(reinterpret_cast<T *>(p.diff), (size_t)p.dim)
                             : const_cast<T *>(sg.in(reinterpret_cast<const T *>(p.diff), (size_t)p.dim));
        if (sg.failed()) return 2;
        hipLaunchKernelGGL((sgd_kernel<T>), dim3(glue_blocks((size_t)p.dim)), dim3(256), 0, state().stream, w, g,
                           (size_t)p.dim, lr, lambda);
        if (!hip_ok(hipGetLastError(), "optimizer launch")) return sg.finish(2);
    }
    return sg.finish(0);
}

// The same update for a list of parameter tensors in one launch: a training step updates dozens of small
// tensors, and one launch each is two microseconds each.
constexpr int SGD_MAXT = 96;  // (3 KB of kernel arguments: the parameter tensors of a ResNet-20 with its normalisation layers are 64)
struct SgdTable {
    void *w[SGD_MAXT], *g[SGD_MAXT];
    unsigned n[SGD_MAXT], first[SGD_MAXT + 1];  // elements; first workgroup of tensor t (first[count] = grid)
    float lr[SGD_MAXT], lambda[SGD_MAXT];
    int count;
};

template <typename T>
__global__ __launch_bounds__(256) void sgd_multi_kernel(const SgdTable t) {
    int k = 0;
    while (k + 1 < t.count && blockIdx.x >= t.first[k + 1]) ++k;
    const size_t i = (size_t)(blockIdx.x - t.first[k]) * 256 + threadIdx.x;
    if (i >= t.n[k]) return;
    T *w = reinterpret_cast<T *>(t.w[k]), *g = reinterpret_cast<T *>(t.g[k]);
    const float lr = t.lr[k], lambda = t.lambda[k];
    float gi = (float)g[i], wi = (float)w[i];
    if (lambda != 0.f) {
        gi = gi + lambda * wi;
        g[i] = (T)gi;
        gi = (float)(T)gi;
    }
    w[i] = (T)(wi - lr * gi);
}

template <typename T, typename Args>
static int sgd_multi(const Args *list, int count, const char *fn) {
    if (count <= 0) return 0;
    if (!list) return glue_bad(fn, "invalid arguments");
    if (!ensure_init()) return 2;
    Stager sg;
    SgdTable t;
    t.count = 0;
    unsigned blocks = 0;
    auto flush = [&]() {
        if (t.count == 0) return true;
        t.first[t.count] = blocks;
        hipLaunchKernelGGL((sgd_multi_kernel<T>), dim3(blocks), dim3(256), 0, state().stream, t);
        t.count = 0;
        blocks = 0;
        return hip_ok(hipGetLastError(), "optimizer launch");
    };
    for (int i = 0; i < count; ++i) {
        const Args &a = list[i];
        if (!a.weights) return glue_bad(fn, "invalid arguments");
        if (a.use_biases == 1 && !a.biases) return glue_bad(fn, "use_biases=1 with a null bias blob");
        for (int part = 0; part < 2; ++part) {
            if (part == 1 && a.use_biases != 1) continue;
            const auto *b = part == 0 ? a.weights : a.biases;
            if (b->dim <= 0) continue;
            if (!b->data || !b->diff) return glue_bad(fn, "null buffer");
            if (t.count == SGD_MAXT && !flush()) return sg.finish(2);
            const float lam = (float)a.weight_decay_lambda;
            t.w[t.count] = sg.inout(reinterpret_cast<T *>(b->data), (size_t)b->dim);
            t.g[t.count] = lam != 0.f ? sg.inout(reinterpret_cast<T *>(b->diff), (size_t)b->dim)
                                      : const_cast<T *>(sg.in(reinterpret_cast<const T *>(b->diff), (size_t)b->dim));
            if (sg.failed()) return 2;
            t.n[t.count] = (unsigned)b->dim;
            t.first[t.count] = blocks;
            t.lr[t.count] = (float)a.learning_rate;
            t.lambda[t.count] = (float)a.weight_decay_lambda;
            blocks += glue_blocks((size_t)b->dim);
            ++t.count;
        }
    }
    return sg.finish(flush() ? 0 : 2);
}

// ---- Batch normalisation (forward: lib/sources/pulp_batchnorm_fp32.c:34-114) ---------------------------
// Statistics per channel over B x H x W, in two launches so that a few channels still fill the chip:
//   1. partial sums per (channel, group of samples): forward x and x^2; backward also dy and dy*x;
//   2. the workgroups of the second kernel own the same (channel, group of samples) pieces, add the channel's
//      partials in a fixed order, form mean and deviation the way the reference does and map their planes.
// The backward pass (the reference has none; the usual one for the forward above):
//   xh = (x - mean) / sd,  dbeta = sum dy,  dgamma = sum dy * xh = (sum dy*x - mean * sum dy) / sd,
//   dx = gamma / sd * (dy - dbeta / n - xh * dgamma / n).
constexpr int BN_SUMS = 4;

template <typename T>
union BnVec {
    uint4 raw;
    T e[16 / sizeof(T)];
};

// What a residual block puts behind a normalisation layer, done in the same kernels:
//   forward   out = [relu](bn(x) [+ skip]);
//   backward  g = (dy [+ dy2]) [where out > 0, else 0], rounded to T like a tensor an element-wise layer would have
//             written; g is the gradient of the normalisation's output and of the skip input (stored to gout when
//             wanted), dx = bn'(g).
template <typename T>
struct BnFuse {
    const T *skip;  // forward: added after the normalisation
    const T *out;   // backward: the forward result (sign = ReLU mask)
    const T *dy2;   // backward: second incoming gradient
    T *gout;        // backward: receives g
    int relu;
    unsigned hw_magic;  // ceil(2^32 / HW) when indices and HW are below 2^16 (sample index by multiplication), else 0
    // backward, second kernel: the sums of the gradient and of gradient * input come from here ([channel][part][4],
    // places 0 and 1) instead of from places 2 and 3 of the first kernel's partials; NULL: from the first kernel
    const float *part_g;
    int nparts_g;
};

template <typename T, bool BW, bool FUSED = false>
__global__ __launch_bounds__(256) void bn_sums_kernel(const T *__restrict__ x, const T *__restrict__ dy,
                                                      float *__restrict__ part, int B, int C, int HW, int per_group,
                                                      int vec, const BnFuse<T> f = BnFuse<T>()) {
    __shared__ float red[BN_SUMS][4];
    const int c = blockIdx.x, grp = blockIdx.y, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    // the group's planes of this channel as one index range: element i = (sample i / HW, position i % HW), so that
    // small planes still keep every thread busy
    const int b0 = grp * per_group, nb = min(B, b0 + per_group) - b0;
    const int total = nb * HW;
    constexpr int VEC = 16 / (int)sizeof(T);
    float s[BN_SUMS] = {0.f, 0.f, 0.f, 0.f};
    if (vec) {  // planes are whole 16-byte vectors
        for (int i = tid * VEC; i < total; i += 256 * VEC) {
            const int bl = f.hw_magic ? (int)__umulhi((unsigned)i, f.hw_magic) : i / HW, e = i - bl * HW;
            const size_t at = ((size_t)(b0 + bl) * C + c) * HW + e;
            BnVec<T> xv, gv;
            xv.raw = *reinterpret_cast<const uint4 *>(x + at);
            if (BW) gv.raw = *reinterpret_cast<const uint4 *>(dy + at);
            if (BW && FUSED) {
                BnVec<T> g2, ov;
                if (f.dy2) {
                    g2.raw = *reinterpret_cast<const uint4 *>(f.dy2 + at);
#pragma unroll
                    for (int q = 0; q < VEC; ++q) gv.e[q] = (T)((float)gv.e[q] + (float)g2.e[q]);
                }
                if (f.relu) {
                    ov.raw = *reinterpret_cast<const uint4 *>(f.out + at);
#pragma unroll
                    for (int q = 0; q < VEC; ++q) gv.e[q] = (float)ov.e[q] > 0.f ? gv.e[q] : (T)0;
                }
                if (f.gout) *reinterpret_cast<uint4 *>(f.gout + at) = gv.raw;
            }
#pragma unroll
            for (int q = 0; q < VEC; ++q) {
                const float v = (float)xv.e[q];
                s[0] += v;
                s[1] += v * v;
                if (BW) {
                    const float g = (float)gv.e[q];
                    s[2] += g;
                    s[3] += g * v;
                }
            }
        }
    } else {
        for (int i = tid; i < total; i += 256) {
            const int bl = f.hw_magic ? (int)__umulhi((unsigned)i, f.hw_magic) : i / HW, e = i - bl * HW;
            const size_t at = ((size_t)(b0 + bl) * C + c) * HW + e;
            const float v = (float)x[at];
            s[0] += v;
            s[1] += v * v;
            if (BW) {
                T gt = dy[at];
                if (FUSED) {
                    if (f.dy2) gt = (T)((float)gt + (float)f.dy2[at]);
                    if (f.relu && !((float)f.out[at] > 0.f)) gt = (T)0;
                    if (f.gout) f.gout[at] = gt;
                }
                const float g = (float)gt;
                s[2] += g;
                s[3] += g * v;
            }
        }
    }
#pragma unroll
    for (int k = 0; k < (BW ? 4 : 2); ++k) {
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) s[k] += __shfl_xor(s[k], off);
        if (lane == 0) red[k][wave] = s[k];
    }
    __syncthreads();
    if (tid < (BW ? 4 : 2))
        part[((size_t)c * gridDim.y + grp) * BN_SUMS + tid] = (red[tid][0] + red[tid][1]) + (red[tid][2] + red[tid][3]);
}

template <typename T, bool BW, bool FUSED = false>
__global__ __launch_bounds__(256) void bn_apply_kernel(const T *__restrict__ x, const T *__restrict__ dy,
                                                       T *__restrict__ out, const T *__restrict__ weight,
                                                       const T *__restrict__ bias, const T *__restrict__ eps,
                                                       const float *__restrict__ part, T *__restrict__ dgamma,
                                                       T *__restrict__ dbeta, int B, int C, int HW, int nparts,
                                                       int per_group, int write_dx, int vec,
                                                       const BnFuse<T> f = BnFuse<T>()) {
    constexpr int VEC = 16 / (int)sizeof(T);
    const int c = blockIdx.x, grp = blockIdx.y, tid = threadIdx.x;
    // the channel's partial sums, folded by the first wave (the order every kernel that needs them keeps)
    __shared__ float tot[BN_SUMS];
    if (tid < 64) {
        float4 v = norm_fold_wave(part, nparts, c, tid);
        if (BW && FUSED && f.part_g) {
            const float4 g = norm_fold_wave(f.part_g, f.nparts_g, c, tid);
            v.z = g.x;
            v.w = g.y;
        }
        if (tid == 0) {
            tot[0] = v.x;
            tot[1] = v.y;
            tot[2] = v.z;
            tot[3] = v.w;
        }
    }
    __syncthreads();
    float s[BN_SUMS] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int k = 0; k < (BW ? 4 : 2); ++k) s[k] = tot[k];
    const float cnt = (float)B * (float)HW;
    float mean, sd;
    norm_mean_sd(s[0], s[1], cnt, (float)eps[0], mean, sd);
    const float w = (float)weight[c];
    const float bb = BW ? 0.f : (float)bias[c];
    const float db = s[2], dg = (s[3] - mean * s[2]) / sd;
    if (BW && grp == 0 && tid == 0) {
        if (dgamma) dgamma[c] = (T)dg;
        if (dbeta) dbeta[c] = (T)db;
    }
    if (BW && !write_dx) return;
    const float k0 = w / sd, k1 = db / cnt, k2 = dg / cnt;
    const float gain = w / sd;  // (the forward pass's division once per channel, not per element)
    auto map = [&](float xv, float gv) {
        if (!BW) return norm_forward(xv, mean, gain, bb);
        const float xh = (xv - mean) / sd;
        return k0 * (gv - k1 - xh * k2);
    };
    // the group's planes of this channel as one index range: element i = (sample i / HW, position i % HW)
    const int b0 = grp * per_group, nb = min(B, b0 + per_group) - b0;
    const int total = nb * HW;
    if (vec) {
        for (int i = tid * VEC; i < total; i += 256 * VEC) {
            const int bl = f.hw_magic ? (int)__umulhi((unsigned)i, f.hw_magic) : i / HW, e = i - bl * HW;
            const size_t at = ((size_t)(b0 + bl) * C + c) * HW + e;
            BnVec<T> xv, gv;
            xv.raw = *reinterpret_cast<const uint4 *>(x + at);
            if (BW) {
                // the gradient the first kernel formed (stored, or formed again the same way)
                gv.raw = *reinterpret_cast<const uint4 *>((FUSED && f.gout ? f.gout : dy) + at);
                if (FUSED && !f.gout) {
                    BnVec<T> g2, ov;
                    if (f.dy2) {
                        g2.raw = *reinterpret_cast<const uint4 *>(f.dy2 + at);
#pragma unroll
                        for (int q = 0; q < VEC; ++q) gv.e[q] = (T)((float)gv.e[q] + (float)g2.e[q]);
                    }
                    if (f.relu) {
                        ov.raw = *reinterpret_cast<const uint4 *>(f.out + at);
#pragma unroll
                        for (int q = 0; q < VEC; ++q) gv.e[q] = (float)ov.e[q] > 0.f ? gv.e[q] : (T)0;
                    }
                }
            }
            if (!BW && FUSED) {
                BnVec<T> sv;
                if (f.skip) sv.raw = *reinterpret_cast<const uint4 *>(f.skip + at);
#pragma unroll
                for (int q = 0; q < VEC; ++q) {
                    float v = map((float)xv.e[q], 0.f);
                    if (f.skip) v += (float)sv.e[q];
                    if (f.relu) v = fmaxf(v, 0.f);
                    xv.e[q] = (T)v;
                }
            } else {
#pragma unroll
                for (int q = 0; q < VEC; ++q) xv.e[q] = (T)map((float)xv.e[q], BW ? (float)gv.e[q] : 0.f);
            }
            *reinterpret_cast<uint4 *>(out + at) = xv.raw;
        }
    } else {
        for (int i = tid; i < total; i += 256) {
            const int bl = f.hw_magic ? (int)__umulhi((unsigned)i, f.hw_magic) : i / HW, e = i - bl * HW;
            const size_t at = ((size_t)(b0 + bl) * C + c) * HW + e;
            if (!BW && FUSED) {
                float v = map((float)x[at], 0.f);
                if (f.skip) v += (float)f.skip[at];
                if (f.relu) v = fmaxf(v, 0.f);
                out[at] = (T)v;
                continue;
            }
            T gt = BW ? (FUSED && f.gout ? f.gout[at] : dy[at]) : (T)0;
            if (BW && FUSED && !f.gout) {
                if (f.dy2) gt = (T)((float)gt + (float)f.dy2[at]);
                if (f.relu && !((float)f.out[at] > 0.f)) gt = (T)0;
            }
            out[at] = (T)map((float)x[at], (float)gt);
        }
    }
}

// `given`: sums of the input left by the convolution before (used when they cover this tensor).
// `given_g` (backward): sums of the gradient and of gradient * input left by the convolution behind, which has also
// formed the gradient itself in output->diff; valid ones switch the fusion off (nothing is added or masked again).
template <typename T, typename Args, typename Fusion = void>
static int batch_norm_step(const Args *a, int bw, const char *fn, const Fusion *fu = nullptr,
                           const ::ptl_norm_stats *given = nullptr, const ::ptl_norm_stats *given_g = nullptr) {
    constexpr bool FUSED = !std::is_void<Fusion>::value;
    if (!a || !a->input || !a->output || !a->weight_data || !a->eps || (!bw && !a->bias_data) || (FUSED && !fu))
        return glue_bad(fn, "invalid arguments");
    if (a->B <= 0 || a->C <= 0 || a->H <= 0 || a->W <= 0) return glue_bad(fn, "invalid tensor geometry");
    if (!ensure_init()) return 2;
    State &st = state();
    const int B = a->B, C = a->C, HW = a->H * a->W;
    const size_t n = (size_t)B * C * HW;
    if ((size_t)B * C >= ((size_t)1 << 31)) return glue_bad(fn, "too many planes");
    // groups of samples: about four workgroups per CU - two for tensors of a few megabytes, whose launches are over
    // before more of them would have started (the 21 + 3 normalisation launches of a ResNet-20 step at batch 128:
    // 8 us less per step, measured side by side with one, three, four and eight per CU)
    const int per_cu = n * sizeof(T) <= ((size_t)16 << 20) ? 2 : 4;
    int groups = (per_cu * st.num_cu + C - 1) / C;
    if (groups > 64) groups = 64;  // (more only lengthens the second kernel's fold)
    if (groups > B) groups = B;
    const int per_group = (B + groups - 1) / groups;
    groups = (B + per_group - 1) / per_group;
    const unsigned hw_magic = (HW > 1 && HW < 65536 && (long long)per_group * HW + 4096 < 65536)
                                  ? (unsigned)((((unsigned long long)1 << 32) + HW - 1) / HW)
                                  : 0u;
    BnFuse<T> f0 = {};
    f0.hw_magic = hw_magic;
    float *part = workspace((size_t)C * groups * BN_SUMS * sizeof(float));
    if (!part) return 2;
    Stager sg;
    const T *x = sg.in(reinterpret_cast<const T *>(a->input->data), n);
    const T *w = sg.in(reinterpret_cast<const T *>(a->weight_data), (size_t)C);
    auto aligned16 = [](const void *p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; };
    const int VEC = 16 / (int)sizeof(T);
    const T *eps = sg.in(reinterpret_cast<const T *>(a->eps), (size_t)1);
    if (!x) return glue_bad(fn, "null buffer");
    auto covers = [&](const ::ptl_norm_stats *g) {
        return g && g->valid == 1 && g->part && g->channels == C && g->parts > 0 && g->count == (size_t)B * HW &&
               (size_t)C * g->parts * BN_SUMS * sizeof(float) <= g->bytes && reinterpret_cast<uintptr_t>(g->part) % 16 == 0;
    };
    if (!bw) {
        T *y = sg.out(reinterpret_cast<T *>(a->output->data), n);
        const T *b = sg.in(reinterpret_cast<const T *>(a->bias_data), (size_t)C);
        if (sg.failed() || !y) return sg.failed() ? 2 : glue_bad(fn, "null buffer");
        int vec = HW % VEC == 0 && aligned16(x) && aligned16(y);
        BnFuse<T> f = {};
        f.hw_magic = hw_magic;
        if constexpr (FUSED) {
            f.relu = fu->relu ? 1 : 0;
            f.skip = fu->skip ? sg.in(reinterpret_cast<const T *>(fu->skip), n) : nullptr;
            if (sg.failed()) return 2;
            vec = vec && aligned16(f.skip);
        }
        const bool have = covers(given);
        if (!have)
            hipLaunchKernelGGL((bn_sums_kernel<T, false>), dim3(C, groups), dim3(256), 0, st.stream, x,
                               (const T *)nullptr, part, B, C, HW, per_group, vec, f0);
        hipLaunchKernelGGL((bn_apply_kernel<T, false, FUSED>), dim3(C, groups), dim3(256), 0, st.stream, x,
                           (const T *)nullptr, y, w, b, eps, have ? given->part : part, (T *)nullptr, (T *)nullptr, B,
                           C, HW, have ? given->parts : groups, per_group, 1, vec, f);
    } else {
        const T *dy = sg.in(reinterpret_cast<const T *>(a->output->diff), n);
        const bool want_dx = !a->skip_in_grad, want_dw = !a->skip_wg_grad;
        T *dx = want_dx ? sg.out(reinterpret_cast<T *>(a->input->diff), n) : nullptr;
        T *dg = want_dw && a->coeff ? sg.out(reinterpret_cast<T *>(a->coeff->diff), (size_t)C) : nullptr;
        T *db = want_dw && a->bias ? sg.out(reinterpret_cast<T *>(a->bias->diff), (size_t)C) : nullptr;
        if (sg.failed() || !dy || (want_dx && !dx)) return sg.failed() ? 2 : glue_bad(fn, "null buffer");
        int vec = HW % VEC == 0 && aligned16(x) && aligned16(dy) && (!dx || aligned16(dx));
        BnFuse<T> f = {};
        f.hw_magic = hw_magic;
        const bool formed = FUSED && covers(given_g);  // the gradient in output->diff is final
        if constexpr (FUSED) {
            if (formed && covers(given)) {
                // every sum is there: the second kernel alone
                f.part_g = given_g->part;
                f.nparts_g = given_g->parts;
                hipLaunchKernelGGL((bn_apply_kernel<T, true, FUSED>), dim3(C, want_dx ? groups : 1), dim3(256), 0,
                                   st.stream, x, dy, dx, w, (const T *)nullptr, eps, given->part, dg, db, B, C, HW,
                                   given->parts, per_group, want_dx ? 1 : 0, vec, f);
                return sg.finish(hip_ok(hipGetLastError(), "batch norm launch") ? 0 : 2);
            }
        }
        if constexpr (FUSED) if (!formed) {
            f.relu = fu->relu ? 1 : 0;
            if (f.relu) {
                if (!a->output->data) return glue_bad(fn, "the ReLU mask needs the forward result in output->data");
                f.out = sg.in(reinterpret_cast<const T *>(a->output->data), n);
            }
            f.dy2 = fu->diff2 ? sg.in(reinterpret_cast<const T *>(fu->diff2), n) : nullptr;
            f.gout = fu->skip_diff ? sg.out(reinterpret_cast<T *>(fu->skip_diff), n) : nullptr;
            if (sg.failed()) return 2;
            vec = vec && aligned16(f.out) && aligned16(f.dy2) && aligned16(f.gout);
        }
        hipLaunchKernelGGL((bn_sums_kernel<T, true, FUSED>), dim3(C, groups), dim3(256), 0, st.stream, x, dy, part, B, C,
                           HW, per_group, vec, f);
        // without an input gradient only the first group of every channel runs (it writes dgamma / dbeta)
        hipLaunchKernelGGL((bn_apply_kernel<T, true, FUSED>), dim3(C, want_dx ? groups : 1), dim3(256), 0, st.stream, x,
                           dy, dx, w, (const T *)nullptr, eps, part, dg, db, B, C, HW, groups, per_group,
                           want_dx ? 1 : 0, vec, f);
    }
    return sg.finish(hip_ok(hipGetLastError(), "batch norm launch") ? 0 : 2);
}

}  // namespace ptl

extern "C" {

int ptl_relu_fp32_batched(const struct act_args *a, int ns, int step) {
    return ptl::relu_step<float>(a, ns, step, step ? "pulp_relu_fp32_bw_cl" : "pulp_relu_fp32_fw_cl");
}
int ptl_relu_fp16_batched(const struct act_args_fp16 *a, int ns, int step) {
    return ptl::relu_step<ptl::half_t>(a, ns, step, step ? "pulp_relu_fp16_bw_cl" : "pulp_relu_fp16_fw_cl");
}
int ptl_residual_fp32_batched(const struct SkipConn_args *a, int ns, int step) {
    return ptl::residual_step<float>(
        a, ns, step, step == 0 ? "pulp_residualconn_fp32_fw" : step == 1 ? "pulp_sumnode_fp32_bw" : "pulp_residualconn_fp32_bw");
}
int ptl_residual_fp16_batched(const struct SkipConn_args_fp16 *a, int ns, int step) {
    return ptl::residual_step<ptl::half_t>(
        a, ns, step, step == 0 ? "pulp_residualconn_fp16_fw" : step == 1 ? "pulp_sumnode_fp16_bw" : "pulp_residualconn_fp16_bw");
}
int ptl_avgpool_fp32_batched(const struct pool_args *a, int ns, int step) {
    return ptl::avgpool_step<float>(a, ns, step, step ? "pulp_avgpool_fp32_bw_cl" : "pulp_avgpool_fp32_fw_cl");
}
int ptl_avgpool_fp16_batched(const struct pool_args_fp16 *a, int ns, int step) {
    return ptl::avgpool_step<ptl::half_t>(a, ns, step, step ? "pulp_avgpool_fp16_bw_cl" : "pulp_avgpool_fp16_fw_cl");
}
int ptl_cross_entropy_fp32_batched(const struct loss_args *a, int ns, int step) {
    return ptl::cross_entropy_step<float>(a, ns, step, step ? "pulp_CrossEntropyLoss_backward" : "pulp_CrossEntropyLoss");
}
int ptl_cross_entropy_fp16_batched(const struct loss_args_fp16 *a, int ns, int step) {
    return ptl::cross_entropy_step<ptl::half_t>(a, ns, step,
                                                step ? "pulp_CrossEntropyLoss_backward_fp16" : "pulp_CrossEntropyLoss_fp16");
}
int ptl_pool_linear_loss_fp32_batched(const struct pool_args *pool, const struct Linear_args *lin, const struct loss_args *loss,
                                      int ns, struct ptl_wg_batch *batch) {
    return ptl::head_step<float>(pool, lin, loss, ns, batch, ptl_avgpool_fp32_batched, ptl_linear_fp32_fw_batched,
                                 ptl_linear_fp32_bw_batched, ptl_cross_entropy_fp32_batched, "ptl_pool_linear_loss_fp32_batched");
}
int ptl_pool_linear_loss_fp16_batched(const struct pool_args_fp16 *pool, const struct Linear_args_fp16 *lin,
                                      const struct loss_args_fp16 *loss, int ns, struct ptl_wg_batch *batch) {
    return ptl::head_step<ptl::half_t>(pool, lin, loss, ns, batch, ptl_avgpool_fp16_batched, ptl_linear_fp16_fw_batched,
                                       ptl_linear_fp16_bw_batched, ptl_cross_entropy_fp16_batched,
                                       "ptl_pool_linear_loss_fp16_batched");
}
int ptl_gradient_descent_fp32(const struct optim_args *a) {
    return ptl::sgd_step<float>(a, "pulp_gradient_descent_fp32");
}
int ptl_gradient_descent_fp16(const struct optim_args_fp16 *a) {
    return ptl::sgd_step<ptl::half_t>(a, "pulp_gradient_descent_fp16");
}
int ptl_gradient_descent_fp32_multi(const struct optim_args *list, int count) {
    return ptl::sgd_multi<float>(list, count, "ptl_gradient_descent_fp32_multi");
}
int ptl_gradient_descent_fp16_multi(const struct optim_args_fp16 *list, int count) {
    return ptl::sgd_multi<ptl::half_t>(list, count, "ptl_gradient_descent_fp16_multi");
}
int ptl_batch_norm_fp32_fw(const struct BatchNorm_args_fp32 *a) {
    return ptl::batch_norm_step<float>(a, 0, "pulp_batch_norm_fp32_fw_cl");
}
int ptl_batch_norm_fp32_bw(const struct BatchNorm_args_fp32 *a) {
    return ptl::batch_norm_step<float>(a, 1, "ptl_batch_norm_fp32_bw");
}
int ptl_batch_norm_fp16_fw(const struct BatchNorm_args_fp16 *a) {
    return ptl::batch_norm_step<ptl::half_t>(a, 0, "ptl_batch_norm_fp16_fw");
}
int ptl_batch_norm_fp16_bw(const struct BatchNorm_args_fp16 *a) {
    return ptl::batch_norm_step<ptl::half_t>(a, 1, "ptl_batch_norm_fp16_bw");
}
int ptl_batch_norm_fused_fp32_fw(const struct BatchNorm_args_fp32 *a, const struct ptl_norm_fusion_fp32 *f) {
    return ptl::batch_norm_step<float>(a, 0, "ptl_batch_norm_fused_fp32_fw", f);
}
int ptl_batch_norm_fused_fp32_bw(const struct BatchNorm_args_fp32 *a, const struct ptl_norm_fusion_fp32 *f) {
    return ptl::batch_norm_step<float>(a, 1, "ptl_batch_norm_fused_fp32_bw", f);
}
int ptl_batch_norm_fused_fp16_fw(const struct BatchNorm_args_fp16 *a, const struct ptl_norm_fusion_fp16 *f) {
    return ptl::batch_norm_step<ptl::half_t>(a, 0, "ptl_batch_norm_fused_fp16_fw", f);
}
int ptl_batch_norm_fused_fp16_bw(const struct BatchNorm_args_fp16 *a, const struct ptl_norm_fusion_fp16 *f) {
    return ptl::batch_norm_step<ptl::half_t>(a, 1, "ptl_batch_norm_fused_fp16_bw", f);
}
int ptl_batch_norm_fused_fp32_fw_stats(const struct BatchNorm_args_fp32 *a, const struct ptl_norm_fusion_fp32 *f,
                                       const struct ptl_norm_stats *st) {
    static const struct ptl_norm_fusion_fp32 none = {};
    return ptl::batch_norm_step<float>(a, 0, "ptl_batch_norm_fused_fp32_fw_stats", f ? f : &none, st);
}
int ptl_batch_norm_fused_fp16_fw_stats(const struct BatchNorm_args_fp16 *a, const struct ptl_norm_fusion_fp16 *f,
                                       const struct ptl_norm_stats *st) {
    static const struct ptl_norm_fusion_fp16 none = {};
    return ptl::batch_norm_step<ptl::half_t>(a, 0, "ptl_batch_norm_fused_fp16_fw_stats", f ? f : &none, st);
}

int ptl_batch_norm_fused_fp32_bw_stats(const struct BatchNorm_args_fp32 *a, const struct ptl_norm_fusion_fp32 *f,
                                       const struct ptl_norm_stats *fw, const struct ptl_norm_stats *bw) {
    static const struct ptl_norm_fusion_fp32 none = {};
    return ptl::batch_norm_step<float>(a, 1, "ptl_batch_norm_fused_fp32_bw_stats", f ? f : &none, fw, bw);
}
int ptl_batch_norm_fused_fp16_bw_stats(const struct BatchNorm_args_fp16 *a, const struct ptl_norm_fusion_fp16 *f,
                                       const struct ptl_norm_stats *fw, const struct ptl_norm_stats *bw) {
    static const struct ptl_norm_fusion_fp16 none = {};
    return ptl::batch_norm_step<ptl::half_t>(a, 1, "ptl_batch_norm_fused_fp16_bw_stats", f ? f : &none, fw, bw);
}

}  // extern "C"
