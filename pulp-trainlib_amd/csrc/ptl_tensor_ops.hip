// Bandwidth-bound kernels of the training core: depthwise convolution
// (forward, weight gradient, input gradient), the materialising patch-matrix
// builders (im2row / im2col), weight block transpose, matrix and n-d
// transposition, layout change, padding and the streaming helpers.  All of
// them are index permutations or short stencils over tensors that are read
// and written once, so they are organised for coalesced global access (64
// consecutive lanes touch consecutive addresses on the contiguous side) and
// measured against HBM bandwidth, not the matrix cores.
#include "ptl_common.hpp"
#include "ptl_host.hpp"
#include "ptl_api.h"

#include <stdio.h>

namespace ptl {

static inline unsigned nblocks(size_t n) { return (unsigned)((n + 255) / 256); }

// x / d as a multiplication by m = ceil(2^32 / d): exact for x below 2^16.  d = 1 gives m = 2^32, which a 32-bit
// m holds as 0: that value stands for the identity.
__device__ inline unsigned div_magic(unsigned x, unsigned m) { return m ? __umulhi(x, m) : x; }

// ---- Depthwise convolution (CHW planes, one filter per channel) -----------------
struct DwGeom {
    int C, H, W, Ho, Wo, Hk, Wk;
    int Up, Lp, sh, sw;
};

// Y[b,c,ho,wo] = sum_{hk,wk} W[c,hk,wk] * X[b,c,ho*sh-Up+hk, wo*sw-Lp+wk]
template <typename T>
__global__ __launch_bounds__(256) void dw_fw_kernel(const T *__restrict__ X, const T *__restrict__ Wt,
                                                    T *__restrict__ Y, DwGeom g, size_t total) {
    size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= total) return;
    int wo = (int)(idx % g.Wo);
    size_t t = idx / g.Wo;
    int ho = (int)(t % g.Ho);
    size_t plane = t / g.Ho;  // b*C + c
    int c = (int)(plane % g.C);
    const T *xp = X + plane * g.H * g.W;
    const T *wp = Wt + (size_t)c * g.Hk * g.Wk;
    int h0 = ho * g.sh - g.Up, w0 = wo * g.sw - g.Lp;
    float s = 0.f;
    for (int hk = 0; hk < g.Hk; ++hk) {
        int h = h0 + hk;
        if ((unsigned)h >= (unsigned)g.H) continue;
        for (int wk = 0; wk < g.Wk; ++wk) {
            int w = w0 + wk;
            if ((unsigned)w < (unsigned)g.W) s += (float)wp[hk * g.Wk + wk] * (float)xp[h * g.W + w];
        }
    }
    Y[idx] = (T)s;
}

// dX[b,c,hi,wi] = sum_{hk,wk} W[c,hk,wk] * dY[b,c,ho,wo], ho*sh = hi+Up-hk, wo*sw = wi+Lp-wk
template <typename T>
__global__ __launch_bounds__(256) void dw_ig_kernel(const T *__restrict__ dY, const T *__restrict__ Wt,
                                                    T *__restrict__ dX, DwGeom g, size_t total) {
    size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= total) return;
    int wi = (int)(idx % g.W);
    size_t t = idx / g.W;
    int hi = (int)(t % g.H);
    size_t plane = t / g.H;
    int c = (int)(plane % g.C);
    const T *gp = dY + plane * g.Ho * g.Wo;
    const T *wp = Wt + (size_t)c * g.Hk * g.Wk;
    float s = 0.f;
    for (int hk = 0; hk < g.Hk; ++hk) {
        int hq = hi + g.Up - hk;
        if (hq < 0 || hq % g.sh != 0) continue;
        int ho = hq / g.sh;
        if (ho >= g.Ho) continue;
        for (int wk = 0; wk < g.Wk; ++wk) {
            int wq = wi + g.Lp - wk;
            if (wq < 0 || wq % g.sw != 0) continue;
            int wo = wq / g.sw;
            if (wo < g.Wo) s += (float)wp[hk * g.Wk + wk] * (float)gp[ho * g.Wo + wo];
        }
    }
    dX[idx] = (T)s;
}

// part[chunk][c][tap] = sum over this chunk's (sample, pixel) range of X * dY.
// grid = (C, chunks); every thread keeps all taps of its channel in registers.
template <typename T, int MAXT>
__global__ __launch_bounds__(256) void dw_wg_kernel(const T *__restrict__ X, const T *__restrict__ dY,
                                                    float *__restrict__ part, DwGeom g, int ns, int per_chunk) {
    const int c = blockIdx.x;
    const int P = g.Ho * g.Wo;
    const size_t n = (size_t)ns * P;
    size_t i0 = (size_t)blockIdx.y * per_chunk;
    size_t i1 = i0 + per_chunk < n ? i0 + per_chunk : n;
    const int taps = g.Hk * g.Wk;
    float acc[MAXT];
#pragma unroll
    for (int t = 0; t < MAXT; ++t) acc[t] = 0.f;
    for (size_t i = i0 + threadIdx.x; i < i1; i += 256) {
        int b = (int)(i / P), p = (int)(i % P);
        int ho = p / g.Wo, wo = p % g.Wo;
        size_t plane = (size_t)b * g.C + c;
        float gy = (float)dY[plane * P + p];
        const T *xp = X + plane * g.H * g.W;
        int h0 = ho * g.sh - g.Up, w0 = wo * g.sw - g.Lp;
#pragma unroll
        for (int t = 0; t < MAXT; ++t) {
            if (t < taps) {
                int hk = t / g.Wk, wk = t % g.Wk;
                int h = h0 + hk, w = w0 + wk;
                if ((unsigned)h < (unsigned)g.H && (unsigned)w < (unsigned)g.W)
                    acc[t] += gy * (float)xp[h * g.W + w];
            }
        }
    }
    __shared__ float red[4][MAXT];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
    for (int t = 0; t < MAXT; ++t) {
        float v = acc[t];
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) v += __shfl_down(v, o, 64);
        if (lane == 0) red[wave][t] = v;
    }
    __syncthreads();
    if ((int)threadIdx.x < taps) {
        int t = threadIdx.x;
        float v = red[0][t] + red[1][t] + red[2][t] + red[3][t];
        part[((size_t)blockIdx.y * g.C + c) * taps + t] = v;
    }
}

template <typename T>
__global__ __launch_bounds__(256) void dw_wg_reduce_kernel(const float *__restrict__ part, T *__restrict__ dW,
                                                           int n, int chunks) {
    int i = blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    float s = 0.f;
    for (int z = 0; z < chunks; ++z) s += part[(size_t)z * n + i];
    dW[i] = (T)s;
}


// ---- Depthwise fast path: unit stride, KxK with K = 3 or 5, rows at least 32 wide ------
// Lanes run along a row (consecutive lanes = consecutive columns, so every global access
// of a wave is one contiguous run); each thread owns a column strip of RB output rows and
// walks down the input rows once, keeping the K horizontally shifted values of the current
// input row in registers.  Per output element this is (RB+K-1)*K/RB loads instead of K*K.
constexpr int DW_RB = 8;  // output rows per thread

// The K column shifts of one source row for this lane's column c: v[j] = row[c + j - pl] (zero
// outside the row).  One load of the lane's own column, the shifts come from the neighbouring
// lanes; only lanes at the edge of the wave's 64-column chunk load their missing neighbours.
template <typename T, int K>
__device__ inline void dw_row_shifts(const T *__restrict__ row, bool rowok, int c, int lane, int pl, int Ws,
                                     const bool (&colok)[K], float (&v)[K]) {
    const float own = (rowok && (unsigned)c < (unsigned)Ws) ? (float)row[c] : 0.f;
#pragma unroll
    for (int j = 0; j < K; ++j) {
        const int d = j - pl;
        const float nb = __shfl(own, lane + d, 64);
        const bool in_wave = (unsigned)(lane + d) < 64u;
        float val = in_wave ? nb : 0.f;
        if (!in_wave && rowok && colok[j]) val = (float)row[c + d];
        v[j] = (d == 0) ? own : val;
    }
}


// out[p][r][c] = sum_{i,j} wt[ch][i][j] * in[p][r + i - pu][c + j - pl], zero outside the source.
// FLIP uses wt[K-1-i][K-1-j]: with pu = K-1-Up, pl = K-1-Lp and the output gradient as
// source this is the input gradient.
template <typename T, int K, bool FLIP>
__global__ __launch_bounds__(256) void dw_rows_kernel(const T *__restrict__ src, const T *__restrict__ Wt,
                                                      T *__restrict__ dst, int C, int Hs, int Ws, int Hd, int Wd,
                                                      int pu, int pl, int row_blocks, int col_chunks, long total_waves) {
    long wave = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (wave >= total_waves) return;
    const int lane = threadIdx.x & 63;
    int cc = (int)(wave % col_chunks);
    long t = wave / col_chunks;
    int rb = (int)(t % row_blocks);
    long plane = t / row_blocks;
    const int ch = (int)(plane % C);
    const int c = cc * 64 + lane;
    const int r0 = rb * DW_RB;
    float w[K][K];
#pragma unroll
    for (int i = 0; i < K; ++i)
#pragma unroll
        for (int j = 0; j < K; ++j)
            w[i][j] = (float)Wt[(size_t)ch * K * K + (FLIP ? (K - 1 - i) * K + (K - 1 - j) : i * K + j)];
    float acc[DW_RB];
#pragma unroll
    for (int q = 0; q < DW_RB; ++q) acc[q] = 0.f;
    const T *sp = src + (size_t)plane * Hs * Ws;
    bool colok[K];
#pragma unroll
    for (int j = 0; j < K; ++j) colok[j] = (unsigned)(c + j - pl) < (unsigned)Ws;
#pragma unroll
    for (int rr = 0; rr < DW_RB + K - 1; ++rr) {
        const int h = r0 + rr - pu;  // source row (wave-uniform)
        float v[K];
        const bool rowok = (unsigned)h < (unsigned)Hs;
        dw_row_shifts<T, K>(sp + (size_t)(rowok ? h : 0) * Ws, rowok, c, lane, pl, Ws, colok, v);
#pragma unroll
        for (int i = 0; i < K; ++i) {
            const int q = rr - i;  // output row (relative) fed by this source row through tap row i
            if (q >= 0 && q < DW_RB) {
#pragma unroll
                for (int j = 0; j < K; ++j) acc[q] += w[i][j] * v[j];
            }
        }
    }
    if (c < Wd) {
        T *dp = dst + (size_t)plane * Hd * Wd;
#pragma unroll
        for (int q = 0; q < DW_RB; ++q)
            if (r0 + q < Hd) dp[(size_t)(r0 + q) * Wd + c] = (T)acc[q];
    }
}

// Weight gradient, same walk: part[wave][i][j] = sum over this wave's strip of
// X[r + i - pu][c + j - pl] * dY[r][c]; a wave owns (plane, row block, column chunk).
// Partials are summed per channel by dw_wg_reduce_kernel2.
template <typename T, int K>
__global__ __launch_bounds__(256) void dw_wg_rows_kernel(const T *__restrict__ X, const T *__restrict__ dY,
                                                         float *__restrict__ part, int C, int H, int W, int Ho, int Wo,
                                                         int pu, int pl, int row_blocks, int col_chunks, int rows_per,
                                                         long total_waves) {
    long wave = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (wave >= total_waves) return;
    const int lane = threadIdx.x & 63;
    int cc = (int)(wave % col_chunks);
    long t = wave / col_chunks;
    int rb = (int)(t % row_blocks);
    long plane = t / row_blocks;
    const int c = cc * 64 + lane;
    const int r0 = rb * rows_per;
    const int r1 = min(Ho, r0 + rows_per);
    float acc[K][K];
#pragma unroll
    for (int i = 0; i < K; ++i)
#pragma unroll
        for (int j = 0; j < K; ++j) acc[i][j] = 0.f;
    const T *xp = X + (size_t)plane * H * W;
    const T *gp = dY + (size_t)plane * Ho * Wo;
    bool colok[K];
#pragma unroll
    for (int j = 0; j < K; ++j) colok[j] = (unsigned)(c + j - pl) < (unsigned)W;
    const bool gcol = c < Wo;
    // sliding window of K source rows (each at K column shifts)
    float win[K][K];
#pragma unroll
    for (int i = 0; i < K - 1; ++i) {
        const int h = r0 + i - pu;
        const bool rowok = (unsigned)h < (unsigned)H;
        dw_row_shifts<T, K>(xp + (size_t)(rowok ? h : 0) * W, rowok, c, lane, pl, W, colok, win[i]);
    }
    for (int r = r0; r < r1; ++r) {
        const int h = r + (K - 1) - pu;
        const bool rowok = (unsigned)h < (unsigned)H;
        dw_row_shifts<T, K>(xp + (size_t)(rowok ? h : 0) * W, rowok, c, lane, pl, W, colok, win[K - 1]);
        const float g = gcol ? (float)gp[(size_t)r * Wo + c] : 0.f;
#pragma unroll
        for (int i = 0; i < K; ++i)
#pragma unroll
            for (int j = 0; j < K; ++j) acc[i][j] += win[i][j] * g;
#pragma unroll
        for (int i = 0; i < K - 1; ++i)
#pragma unroll
            for (int j = 0; j < K; ++j) win[i][j] = win[i + 1][j];
    }
#pragma unroll
    for (int i = 0; i < K; ++i)
#pragma unroll
        for (int j = 0; j < K; ++j) {
            float v = acc[i][j];
#pragma unroll
            for (int o = 32; o > 0; o >>= 1) v += __shfl_down(v, o, 64);
            if (lane == 0) part[(size_t)wave * K * K + i * K + j] = v;
        }
}

// dW[ch][tap] = sum over samples b and strips s of part[(b*C + ch)*strips + s][tap]
template <typename T>
__global__ __launch_bounds__(256) void dw_wg_reduce_kernel2(const float *__restrict__ part, T *__restrict__ dW, int ns,
                                                            int C, int strips, int taps) {
    // thread = (tap, slice): consecutive threads read the consecutive taps of one partial; the
    // slices of a tap are folded through LDS in one pass (taps <= 25)
    const int ch = blockIdx.x;
    __shared__ float red[256];
    const int slices = 256 / taps;
    const int tap = threadIdx.x % taps, slice = threadIdx.x / taps;
    float s = 0.f;
    if (slice < slices) {
        for (long i = slice; i < (long)ns * strips; i += slices) {
            long b = i / strips, st = i % strips;
            s += part[(((size_t)b * C + ch) * strips + st) * taps + tap];
        }
    }
    red[threadIdx.x] = s;
    __syncthreads();
    if ((int)threadIdx.x < taps) {
        float t = 0.f;
        for (int k = 0; k < slices; ++k) t += red[k * taps + threadIdx.x];
        dW[(size_t)ch * taps + threadIdx.x] = (T)t;
    }
}

// ---- Depthwise, plane-resident path: unit stride, 3x3 / 5x5, planes that fit LDS ------------------------
// One workgroup per (sample, channel) plane.  The source plane comes in as flat 16-byte loads starting at the
// 16-byte aligned address at or below its first element (a plane of odd size starts anywhere; an aligned
// vector that overlaps the tensor by one byte lies in a mapped page), every thread then produces runs of eight
// consecutive outputs of a row from LDS and stores them as one vector where the destination allows.  Per
// plane this is a handful of 16-byte global instructions instead of one 2-byte access per element and lane.
template <typename T>
__device__ inline const T *dw_load_plane(const T *__restrict__ plane, int elems, uint4 *img, int tid) {
    constexpr int VEC = 16 / (int)sizeof(T);
    const uintptr_t a0 = reinterpret_cast<uintptr_t>(plane);
    const int shift = (int)(a0 & 15) / (int)sizeof(T);
    const uint4 *base = reinterpret_cast<const uint4 *>(a0 & ~(uintptr_t)15);
    const int nvec = (shift + elems + VEC - 1) / VEC;
    for (int v = tid; v < nvec; v += (int)blockDim.x) img[v] = base[v];
    return reinterpret_cast<const T *>(img) + shift;
}

template <typename T>
__device__ inline void dw_store8(T *__restrict__ dst, const float (&acc)[8], int valid) {
    if (valid == 8 && (reinterpret_cast<uintptr_t>(dst) & 3) == 0) {
        union {
            uint4 v[sizeof(T) == 2 ? 1 : 2];
            T e[8];
        } u;
#pragma unroll
        for (int q = 0; q < 8; ++q) u.e[q] = (T)acc[q];
#pragma unroll
        for (int k = 0; k < (sizeof(T) == 2 ? 1 : 2); ++k) reinterpret_cast<uint4 *>(dst)[k] = u.v[k];
    } else {
#pragma unroll
        for (int q = 0; q < 8; ++q)
            if (q < valid) dst[q] = (T)acc[q];
    }
}

// The 8 + K - 1 source values of row h that feed eight outputs starting at column c0 (zero outside the plane).
template <typename T, int K>
__device__ inline void dw_plane_row(const T *img, int h, int Ws, int c0, int pl, float (&v)[8 + K - 1]) {
    const int cf = c0 - pl;
    if (cf >= 0 && cf + 8 + K - 1 <= Ws) {
        const T *row = img + h * Ws + cf;
#pragma unroll
        for (int t = 0; t < 8 + K - 1; ++t) v[t] = (float)row[t];
    } else {
#pragma unroll
        for (int t = 0; t < 8 + K - 1; ++t) v[t] = (unsigned)(cf + t) < (unsigned)Ws ? (float)img[h * Ws + cf + t] : 0.f;
    }
}

// out[p][r][c] = sum_{i,j} wt[ch][i][j] * in[p][r + i - pu][c + j - pl], zero outside the source; FLIP as in
// dw_rows_kernel (input gradient).
template <typename T, int K, bool FLIP>
__global__ __launch_bounds__(256) void dw_plane_kernel(const T *__restrict__ src, const T *__restrict__ Wt,
                                                       T *__restrict__ dst, int C, int Hs, int Ws, int Hd, int Wd,
                                                       int pu, int pl) {
    extern __shared__ uint4 dw_img[];
    const size_t plane = blockIdx.x;
    const int ch = (int)(plane % C), tid = threadIdx.x;
    const T *img = dw_load_plane<T>(src + plane * Hs * Ws, Hs * Ws, dw_img, tid);
    float w[K][K];
#pragma unroll
    for (int i = 0; i < K; ++i)
#pragma unroll
        for (int j = 0; j < K; ++j)
            w[i][j] = (float)Wt[(size_t)ch * K * K + (FLIP ? (K - 1 - i) * K + (K - 1 - j) : i * K + j)];
    __syncthreads();
    const int groups = (Wd + 7) >> 3;
    T *dp = dst + plane * Hd * Wd;
    for (int item = tid; item < Hd * groups; item += 256) {
        const int r = item / groups, c0 = (item - r * groups) * 8;
        float acc[8];
#pragma unroll
        for (int q = 0; q < 8; ++q) acc[q] = 0.f;
#pragma unroll
        for (int i = 0; i < K; ++i) {
            const int h = r + i - pu;
            if ((unsigned)h >= (unsigned)Hs) continue;
            float v[8 + K - 1];
            dw_plane_row<T, K>(img, h, Ws, c0, pl, v);
#pragma unroll
            for (int j = 0; j < K; ++j)
#pragma unroll
                for (int q = 0; q < 8; ++q) acc[q] += w[i][j] * v[q + j];
        }
        dw_store8<T>(dp + (size_t)r * Wd + c0, acc, min(8, Wd - c0));
    }
}

// fp16 planes whose rows can be read two elements at a time (even row length, even column offset, plane start
// 4-byte aligned): a row segment comes from LDS as dwords = pairs of neighbours, and a filter row meets it as
// two-element dot products with fp32 accumulation (v_dot2_f32_f16) plus one mixed-precision FMA for the odd tap -
// about half the vector instructions of the element-wise form, which is what bounds these kernels.
typedef _Float16 dw_h2 __attribute__((ext_vector_type(2)));

// Dwords P[m] = elements (cf + 2m, cf + 2m + 1) of row h, m < NP; zero outside the row.
template <int NP>
__device__ inline void dw_row_pairs(const half_t *img, int h, int Ws, int cf, unsigned (&P)[NP]) {
    const unsigned *row = reinterpret_cast<const unsigned *>(img + h * Ws + cf);
    if (cf >= 0 && cf + 2 * NP <= Ws) {
#pragma unroll
        for (int m = 0; m < NP; ++m) P[m] = row[m];
    } else {
#pragma unroll
        for (int m = 0; m < NP; ++m) P[m] = (unsigned)(cf + 2 * m) < (unsigned)Ws ? row[m] : 0u;
    }
}

// acc[q] += sum_j w[j] * x[q + j] for q < 8, x = the elements of P.  we[m] = (w[2m], w[2m+1]),
// wo[m] = (w[2m+1], w[2m+2]); wf = the taps in fp32.
template <int K>
__device__ inline void dw_row_taps(const unsigned (&P)[(8 + K) / 2], const dw_h2 (&we)[K / 2], const dw_h2 (&wo)[K / 2],
                                   const float (&wf)[K], float (&acc)[8]) {
#pragma unroll
    for (int q = 0; q < 8; ++q) {
        float a = acc[q];
        if ((q & 1) == 0) {
#pragma unroll
            for (int m = 0; m < K / 2; ++m)
                a = __builtin_amdgcn_fdot2(__builtin_bit_cast(dw_h2, P[q / 2 + m]), we[m], a, false);
            if (K & 1) a = fmaf((float)__builtin_bit_cast(dw_h2, P[(q + K - 1) / 2]).x, wf[K - 1], a);
        } else {
            a = fmaf((float)__builtin_bit_cast(dw_h2, P[(q - 1) / 2]).y, wf[0], a);
#pragma unroll
            for (int m = 0; m < (K - 1) / 2; ++m)
                a = __builtin_amdgcn_fdot2(__builtin_bit_cast(dw_h2, P[(q + 1) / 2 + m]), wo[m], a, false);
            if (!(K & 1)) a = fmaf((float)__builtin_bit_cast(dw_h2, P[(q + K - 1) / 2]).x, wf[K - 1], a);
        }
        acc[q] = a;
    }
}

// One workgroup (two waves) per plane; a thread produces a block of RB rows x 8 columns: an input row segment is
// read from LDS once and feeds the (up to K) output rows it belongs to, and the index arithmetic is paid once per
// block instead of once per eight outputs.
template <int K, bool FLIP, int RB = 4, int NT = 128>
__global__ __launch_bounds__(NT) void dw_plane_pairs_kernel(const half_t *__restrict__ src,
                                                             const half_t *__restrict__ Wt, half_t *__restrict__ dst,
                                                             int C, int Hs, int Ws, int Hd, int Wd, int pu, int pl) {
    constexpr int NP = (8 + K) / 2;
    extern __shared__ uint4 dw_img[];
    const size_t plane = blockIdx.x;
    const int ch = (int)(plane % C), tid = threadIdx.x;
    const half_t *img = dw_load_plane<half_t>(src + plane * Hs * Ws, Hs * Ws, dw_img, tid);
    dw_h2 we[K][K / 2], wo[K][K / 2];
    float wf[K][K];
#pragma unroll
    for (int i = 0; i < K; ++i) {
        half_t wr[K];
#pragma unroll
        for (int j = 0; j < K; ++j) {
            wr[j] = Wt[(size_t)ch * K * K + (FLIP ? (K - 1 - i) * K + (K - 1 - j) : i * K + j)];
            wf[i][j] = (float)wr[j];
        }
#pragma unroll
        for (int m = 0; m < K / 2; ++m) {
            we[i][m] = dw_h2{wr[2 * m], wr[2 * m + 1]};
            wo[i][m] = dw_h2{wr[2 * m + 1], wr[(2 * m + 2 < K) ? 2 * m + 2 : K - 1]};
        }
    }
    __syncthreads();
    const int groups = (Wd + 7) >> 3, rblocks = (Hd + RB - 1) / RB;
    half_t *dp = dst + plane * Hd * Wd;
    for (int item = tid; item < rblocks * groups; item += NT) {
        const int rb = item / groups, c0 = (item - rb * groups) * 8, r0 = rb * RB;
        float acc[RB][8];
#pragma unroll
        for (int r = 0; r < RB; ++r)
#pragma unroll
            for (int q = 0; q < 8; ++q) acc[r][q] = 0.f;
#pragma unroll
        for (int hr = 0; hr < RB + K - 1; ++hr) {  // source row r0 - pu + hr feeds output rows r0 + hr - i, i < K
            const int h = r0 + hr - pu;
            if ((unsigned)h >= (unsigned)Hs) continue;
            unsigned P[NP];
            dw_row_pairs<NP>(img, h, Ws, c0 - pl, P);
#pragma unroll
            for (int i = 0; i < K; ++i)
                if (hr - i >= 0 && hr - i < RB) dw_row_taps<K>(P, we[i], wo[i], wf[i], acc[hr - i]);
        }
        const int valid = min(8, Wd - c0);
#pragma unroll
        for (int r = 0; r < RB; ++r)
            if (r0 + r < Hd) dw_store8<half_t>(dp + (size_t)(r0 + r) * Wd + c0, acc[r], valid);
    }
}

// part[group][ch][i][j] = sum over the planes (b, ch) of the samples b of a group of
// X[r + i - pu][c + j - pl] * dY[r][c].  A workgroup owns (channel, sample group), walks the group's planes with
// per-thread sums in registers and reduces once at the end.
template <typename T, int K>
__global__ __launch_bounds__(256) void dw_wg_plane_kernel(const T *__restrict__ X, const T *__restrict__ dY,
                                                          float *__restrict__ part, int C, int ns, int per_group,
                                                          int H, int W, int Ho, int Wo, int pu, int pl, int x_vecs,
                                                          T *__restrict__ direct) {
    extern __shared__ uint4 dw_img[];
    __shared__ float red[4][K * K];
    const int ch = blockIdx.x, grp = blockIdx.y;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    float acc[K][K];
#pragma unroll
    for (int i = 0; i < K; ++i)
#pragma unroll
        for (int j = 0; j < K; ++j) acc[i][j] = 0.f;
    const int groups = (Wo + 7) >> 3;
    const int b_end = min(ns, (grp + 1) * per_group);
    for (int b = grp * per_group; b < b_end; ++b) {
        const size_t plane = (size_t)b * C + ch;
        __syncthreads();  // the previous plane has been consumed
        const T *ximg = dw_load_plane<T>(X + plane * H * W, H * W, dw_img, tid);
        const T *gimg = dw_load_plane<T>(dY + plane * Ho * Wo, Ho * Wo, dw_img + x_vecs, tid);
        __syncthreads();
        for (int item = tid; item < Ho * groups; item += 256) {
            const int r = item / groups, c0 = (item - r * groups) * 8;
            float gy[8];
#pragma unroll
            for (int q = 0; q < 8; ++q) gy[q] = c0 + q < Wo ? (float)gimg[r * Wo + c0 + q] : 0.f;
#pragma unroll
            for (int i = 0; i < K; ++i) {
                const int h = r + i - pu;
                if ((unsigned)h >= (unsigned)H) continue;
                float v[8 + K - 1];
                dw_plane_row<T, K>(ximg, h, W, c0, pl, v);
#pragma unroll
                for (int j = 0; j < K; ++j)
#pragma unroll
                    for (int q = 0; q < 8; ++q) acc[i][j] += v[q + j] * gy[q];
            }
        }
    }
#pragma unroll
    for (int i = 0; i < K; ++i)
#pragma unroll
        for (int j = 0; j < K; ++j) {
            float v = acc[i][j];
#pragma unroll
            for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
            if (lane == 0) red[wave][i * K + j] = v;
        }
    __syncthreads();
    if (tid < K * K) {
        const float sum = (red[0][tid] + red[1][tid]) + (red[2][tid] + red[3][tid]);
        if (direct)  // a single group of samples: this is the gradient itself
            direct[(size_t)ch * K * K + tid] = (decltype(direct[0] + direct[0]))sum;
        else
            part[((size_t)grp * C + ch) * K * K + tid] = sum;
    }
}

// The weight-gradient kernel above for fp16 planes readable as pairs (even row lengths, even left pad, 4-byte
// aligned tensors): the eight output-gradient values of an item are four pairs G, a source row segment is the
// pairs P (and, for the odd taps, the pairs U that start one element later, made with one funnel shift each), and
// tap (i, j) gathers four two-element dot products per item and row.
template <int K>
__global__ __launch_bounds__(256) void dw_wg_plane_pairs_kernel(const half_t *__restrict__ X,
                                                                const half_t *__restrict__ dY,
                                                                float *__restrict__ part, int C, int ns, int per_group,
                                                                int H, int W, int Ho, int Wo, int pu, int pl,
                                                                int x_vecs, half_t *__restrict__ direct) {
    constexpr int NP = (8 + K) / 2, RB = 2;
    extern __shared__ uint4 dw_img[];
    __shared__ float red[4][K * K];
    const int ch = blockIdx.x, grp = blockIdx.y;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    float acc[K][K];
#pragma unroll
    for (int i = 0; i < K; ++i)
#pragma unroll
        for (int j = 0; j < K; ++j) acc[i][j] = 0.f;
    const int groups = (Wo + 7) >> 3, rblocks = (Ho + RB - 1) / RB;
    const int b_end = min(ns, (grp + 1) * per_group);
    for (int b = grp * per_group; b < b_end; ++b) {
        const size_t plane = (size_t)b * C + ch;
        __syncthreads();  // the previous plane has been consumed
        const half_t *ximg = dw_load_plane<half_t>(X + plane * H * W, H * W, dw_img, tid);
        const half_t *gimg = dw_load_plane<half_t>(dY + plane * Ho * Wo, Ho * Wo, dw_img + x_vecs, tid);
        __syncthreads();
        // a thread takes blocks of RB output rows x 8 columns: a source row is read (and its odd-offset pairs made)
        // once for the up to K gradient rows it meets
        for (int item = tid; item < rblocks * groups; item += 256) {
            const int rb = item / groups, c0 = (item - rb * groups) * 8, r0 = rb * RB;
            dw_h2 G[RB][4];
#pragma unroll
            for (int r = 0; r < RB; ++r) {
                const unsigned *grow = reinterpret_cast<const unsigned *>(gimg + (r0 + r) * Wo + c0);
#pragma unroll
                for (int m = 0; m < 4; ++m)
                    G[r][m] = __builtin_bit_cast(dw_h2, (r0 + r < Ho && c0 + 2 * m < Wo) ? grow[m] : 0u);
            }
#pragma unroll
            for (int hr = 0; hr < RB + K - 1; ++hr) {  // source row r0 - pu + hr meets gradient rows r0 + hr - i
                const int h = r0 + hr - pu;
                if ((unsigned)h >= (unsigned)H) continue;
                unsigned P[NP], U[NP - 1];
                dw_row_pairs<NP>(ximg, h, W, c0 - pl, P);
#pragma unroll
                for (int m = 0; m < NP - 1; ++m) U[m] = __builtin_amdgcn_alignbit(P[m + 1], P[m], 16);
#pragma unroll
                for (int i = 0; i < K; ++i) {
                    if (hr - i < 0 || hr - i >= RB) continue;
#pragma unroll
                    for (int j = 0; j < K; ++j) {
                        float a = acc[i][j];
#pragma unroll
                        for (int m = 0; m < 4; ++m)
                            a = __builtin_amdgcn_fdot2(__builtin_bit_cast(dw_h2, (j & 1) ? U[m + j / 2] : P[m + j / 2]),
                                                       G[hr - i][m], a, false);
                        acc[i][j] = a;
                    }
                }
            }
        }
    }
#pragma unroll
    for (int i = 0; i < K; ++i)
#pragma unroll
        for (int j = 0; j < K; ++j) {
            float v = acc[i][j];
#pragma unroll
            for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
            if (lane == 0) red[wave][i * K + j] = v;
        }
    __syncthreads();
    if (tid < K * K) {
        const float sum = (red[0][tid] + red[1][tid]) + (red[2][tid] + red[3][tid]);
        if (direct)  // a single group of samples: this is the gradient itself
            direct[(size_t)ch * K * K + tid] = (decltype(direct[0] + direct[0]))sum;
        else
            part[((size_t)grp * C + ch) * K * K + tid] = sum;
    }
}

// ---- 3x3 fp16 planes straight from global memory -----------------------------------------------------------
// Rows readable as pairs (see dw_row_pairs).  A lane owns a block of DW_DRB output rows x 8 columns and loads
// the DW_DRB + 2 source row segments it needs itself (one 16-byte and one 4-byte load per row, 4-byte aligned):
// no LDS, no barrier, and the blocks of all planes are dealt to the lanes without gaps (a wave may straddle two
// planes).  Neighbouring lanes overlap by two elements per row and two rows per block, which the L1/L2 absorb:
// the planes cross the HBM interface once.
constexpr int DW_DRB = 7;

// P[hr][m] = elements (cf + 2m, cf + 2m + 1) of source row r0 - pu + hr, zero outside the plane.
template <int ROWS>
__device__ inline void dw_direct_rows(const half_t *__restrict__ sp, int Hs, int Ws, int h0, int cf,
                                      unsigned (&P)[ROWS][5]) {
    const bool inner = cf >= 0 && cf + 10 <= Ws;
#pragma unroll
    for (int hr = 0; hr < ROWS; ++hr) {
        const int h = h0 + hr;
        const unsigned *row = reinterpret_cast<const unsigned *>(sp + h * Ws + cf);
        if ((unsigned)h < (unsigned)Hs) {
            if (inner) {
#pragma unroll
                for (int m = 0; m < 5; ++m) P[hr][m] = row[m];
            } else {
#pragma unroll
                for (int m = 0; m < 5; ++m) P[hr][m] = (unsigned)(cf + 2 * m) < (unsigned)Ws ? row[m] : 0u;
            }
        } else {
#pragma unroll
            for (int m = 0; m < 5; ++m) P[hr][m] = 0u;
        }
    }
}

template <bool FLIP>
__global__ __launch_bounds__(256) void dw_direct_kernel(const half_t *__restrict__ src, const half_t *__restrict__ Wt,
                                                        half_t *__restrict__ dst, int C, int Hs, int Ws, int Hd, int Wd,
                                                        int pu, int pl, int rblocks, int groups, unsigned total) {
    constexpr int RB = DW_DRB;
    const unsigned id = blockIdx.x * 256u + threadIdx.x;
    if (id >= total) return;
    const unsigned per_plane = (unsigned)(rblocks * groups);
    const unsigned plane = id / per_plane, blk = id - plane * per_plane;
    // (the last column group and the last row block are moved back to end with the plane when it has at least one
    // full group / block: they then overlap their neighbours, whose values they repeat, and every store is a whole
    // 16-byte one)
    const int rb = (int)(blk / (unsigned)groups);
    const int c0 = Wd >= 8 ? min((int)(blk - (unsigned)rb * groups) * 8, Wd - 8) : 0;
    const int r0 = Hd >= RB ? min(rb * RB, Hd - RB) : 0;
    const int ch = (int)(plane % (unsigned)C);
    dw_h2 we[3], wo[3];
    float w0[3], w2[3];
#pragma unroll
    for (int i = 0; i < 3; ++i) {
        half_t wr[3];
#pragma unroll
        for (int j = 0; j < 3; ++j) wr[j] = Wt[ch * 9 + (FLIP ? (2 - i) * 3 + (2 - j) : i * 3 + j)];
        we[i] = dw_h2{wr[0], wr[1]};
        wo[i] = dw_h2{wr[1], wr[2]};
        w0[i] = (float)wr[0];
        w2[i] = (float)wr[2];
    }
    unsigned P[RB + 2][5];
    dw_direct_rows<RB + 2>(src + (size_t)plane * Hs * Ws, Hs, Ws, r0 - pu, c0 - pl, P);
    float acc[RB][8];
#pragma unroll
    for (int r = 0; r < RB; ++r)
#pragma unroll
        for (int q = 0; q < 8; ++q) acc[r][q] = 0.f;
#pragma unroll
    for (int hr = 0; hr < RB + 2; ++hr) {
#pragma unroll
        for (int i = 0; i < 3; ++i) {
            const int r = hr - i;
            if (r < 0 || r >= RB) continue;
#pragma unroll
            for (int q = 0; q < 8; ++q) {
                float a = acc[r][q];
                if ((q & 1) == 0) {
                    a = __builtin_amdgcn_fdot2(__builtin_bit_cast(dw_h2, P[hr][q / 2]), we[i], a, false);
                    a = fmaf((float)__builtin_bit_cast(dw_h2, P[hr][q / 2 + 1]).x, w2[i], a);
                } else {
                    a = fmaf((float)__builtin_bit_cast(dw_h2, P[hr][q / 2]).y, w0[i], a);
                    a = __builtin_amdgcn_fdot2(__builtin_bit_cast(dw_h2, P[hr][q / 2 + 1]), wo[i], a, false);
                }
                acc[r][q] = a;
            }
        }
    }
    half_t *dp = dst + (size_t)plane * Hd * Wd;
    const int valid = min(8, Wd - c0);
#pragma unroll
    for (int r = 0; r < RB; ++r) {
        if (r0 + r >= Hd) continue;
        half_t *o = dp + (size_t)(r0 + r) * Wd + c0;
        if (valid == 8) {  // (rows are whole dwords: a 16-byte global store needs no more than 4-byte alignment)
            typedef unsigned u4a __attribute__((ext_vector_type(4), aligned(4)));
            union {
                u4a v;
                half_t e[8];
            } u;
#pragma unroll
            for (int q = 0; q < 8; ++q) u.e[q] = (half_t)acc[r][q];
            *reinterpret_cast<u4a *>(o) = u.v;
        } else {
#pragma unroll
            for (int q = 0; q < 8; ++q)
                if (q < valid) o[q] = (half_t)acc[r][q];
        }
    }
}

// Weight gradient the same way: a wave walks planes (b, ch) of its sample group, a lane takes blocks of DW_DRB
// gradient rows x 8 columns with the source rows they meet, the nine tap sums stay in registers; one reduction
// per workgroup at the end.  part[(grp * C + ch) * 9 + tap], or the gradient itself when there is one group.
__global__ __launch_bounds__(256) void dw_wg_direct_kernel(const half_t *__restrict__ X, const half_t *__restrict__ dY,
                                                           float *__restrict__ part, int C, int ns, int per_group, int H,
                                                           int W, int Ho, int Wo, int pu, int pl,
                                                           half_t *__restrict__ direct) {
    constexpr int RB = DW_DRB;
    __shared__ float red[4][9];
    const int ch = blockIdx.x, grp = blockIdx.y;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    float acc[3][3];
#pragma unroll
    for (int i = 0; i < 3; ++i)
#pragma unroll
        for (int j = 0; j < 3; ++j) acc[i][j] = 0.f;
    const int groups = (Wo + 7) >> 3, rblocks = (Ho + RB - 1) / RB;
    const int b_end = min(ns, (grp + 1) * per_group);
    for (int b = grp * per_group + wave; b < b_end; b += 4) {
        const size_t plane = (size_t)b * C + ch;
        const half_t *xp = X + plane * H * W, *gp = dY + plane * Ho * Wo;
        for (int item = lane; item < rblocks * groups; item += 64) {
            const int rb = item / groups, c0 = (item - rb * groups) * 8, r0 = rb * RB;
            dw_h2 G[RB][4];
#pragma unroll
            for (int r = 0; r < RB; ++r) {
                const unsigned *grow = reinterpret_cast<const unsigned *>(gp + (r0 + r) * Wo + c0);
                if (r0 + r < Ho && c0 + 8 <= Wo) {
#pragma unroll
                    for (int m = 0; m < 4; ++m) G[r][m] = __builtin_bit_cast(dw_h2, grow[m]);
                } else {
#pragma unroll
                    for (int m = 0; m < 4; ++m)
                        G[r][m] = __builtin_bit_cast(dw_h2, (r0 + r < Ho && c0 + 2 * m < Wo) ? grow[m] : 0u);
                }
            }
            unsigned P[RB + 2][5];
            dw_direct_rows<RB + 2>(xp, H, W, r0 - pu, c0 - pl, P);
#pragma unroll
            for (int hr = 0; hr < RB + 2; ++hr) {  // source row r0 - pu + hr meets gradient rows r0 + hr - i
                unsigned U[4];
#pragma unroll
                for (int m = 0; m < 4; ++m) U[m] = __builtin_amdgcn_alignbit(P[hr][m + 1], P[hr][m], 16);
#pragma unroll
                for (int i = 0; i < 3; ++i) {
                    if (hr - i < 0 || hr - i >= RB) continue;
#pragma unroll
                    for (int j = 0; j < 3; ++j) {
                        float a = acc[i][j];
#pragma unroll
                        for (int m = 0; m < 4; ++m)
                            a = __builtin_amdgcn_fdot2(__builtin_bit_cast(dw_h2, j == 1 ? U[m] : P[hr][m + j / 2]),
                                                       G[hr - i][m], a, false);
                        acc[i][j] = a;
                    }
                }
            }
        }
    }
#pragma unroll
    for (int i = 0; i < 3; ++i)
#pragma unroll
        for (int j = 0; j < 3; ++j) {
            float v = acc[i][j];
#pragma unroll
            for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
            if (lane == 0) red[wave][i * 3 + j] = v;
        }
    __syncthreads();
    if (tid < 9) {
        const float sum = (red[0][tid] + red[1][tid]) + (red[2][tid] + red[3][tid]);
        if (direct)
            direct[(size_t)ch * 9 + tid] = (half_t)sum;
        else
            part[((size_t)grp * C + ch) * 9 + tid] = sum;
    }
}

template <typename Args>
static int dw_geom(const Args *a, DwGeom &g, int sh, int sw, const char *fn) {
    if (!a || !a->input || !a->coeff || !a->output) {
        printf("[%s] null argument structure\n", fn);
        set_error("%s: null argument structure", fn);
        return 1;
    }
    g.C = a->input->C;
    g.H = a->input->H;
    g.W = a->input->W;
    g.Ho = a->output->H;
    g.Wo = a->output->W;
    g.Hk = a->coeff->H;
    g.Wk = a->coeff->W;
    g.Up = a->Upad;
    g.Lp = a->Lpad;
    g.sh = sh;
    g.sw = sw;
    int nh = g.H - g.Hk + a->Upad + a->Dpad, nw = g.W - g.Wk + a->Lpad + a->Rpad;
    if (g.C <= 0 || g.H <= 0 || g.W <= 0 || g.Hk <= 0 || g.Wk <= 0 || sh <= 0 || sw <= 0 || nh < 0 || nw < 0 ||
        a->Upad < 0 || a->Dpad < 0 || a->Lpad < 0 || a->Rpad < 0 || a->output->C != g.C) {
        printf("[%s] invalid tensor geometry\n", fn);
        set_error("%s: invalid tensor geometry", fn);
        return 1;
    }
    if (g.Ho != nh / sh + 1 || g.Wo != nw / sw + 1) {
        printf("[%s] output blob is %dx%d but the geometry gives %dx%d\n", fn, g.Ho, g.Wo, nh / sh + 1,
               nw / sw + 1);
        set_error("%s: output blob size does not match the convolution geometry", fn);
        return 1;
    }
    if (g.Hk * g.Wk > 49) {
        printf("[%s] kernels above 49 taps are not supported\n", fn);
        set_error("%s: kernels above 49 taps are not supported", fn);
        return 1;
    }
    return 0;
}

// Plane-resident depthwise product (forward, or input gradient with FLIP).
template <typename T, int K, bool FLIP>
static void launch_dw_plane(const T *src, const T *Wt, T *dst, int C, int Hs, int Ws, int Hd, int Wd, int pu, int pl,
                            long planes, hipStream_t stream) {
    const size_t src_img = (size_t)Hs * Ws * sizeof(T) + 32;
    if constexpr (sizeof(T) == 2) {
        // 3x3 with rows of whole dwords on both sides and at least one group of eight columns: straight from global
        // memory (forward, and the input gradient as the flipped correlation over the output gradient)
        if (K == 3 && Ws % 2 == 0 && Wd % 2 == 0 && Wd >= 8 && pl % 2 == 0 && reinterpret_cast<uintptr_t>(src) % 4 == 0 &&
            reinterpret_cast<uintptr_t>(dst) % 4 == 0) {
            const int rblocks = (Hd + DW_DRB - 1) / DW_DRB, groups = (Wd + 7) / 8;
            const long long total = (long long)planes * rblocks * groups;
            if (total < ((long long)1 << 31)) {
                hipLaunchKernelGGL((dw_direct_kernel<FLIP>), dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream,
                                   src, Wt, dst, C, Hs, Ws, Hd, Wd, pu, pl, rblocks, groups, (unsigned)total);
                return;
            }
        }
        // rows readable as pairs: see dw_plane_pairs_kernel
        if (Ws % 2 == 0 && pl % 2 == 0 && reinterpret_cast<uintptr_t>(src) % 4 == 0) {
            hipLaunchKernelGGL((dw_plane_pairs_kernel<K, FLIP>), dim3((unsigned)planes), dim3(128), src_img, stream, src,
                               Wt, dst, C, Hs, Ws, Hd, Wd, pu, pl);
            return;
        }
    }
    hipLaunchKernelGGL((dw_plane_kernel<T, K, FLIP>), dim3((unsigned)planes), dim3(256), src_img, stream, src, Wt, dst,
                       C, Hs, Ws, Hd, Wd, pu, pl);
}

// ---- partial sums of the allocation-free weight-gradient entry point ---------------------------------
// A fixed array in device memory, one copy per GPU, held until the process ends.  In host code the array's
// name is only a handle: its device address is looked up once per device (dw_noalloc_setup, called from the
// library's init) and that pointer is what kernels receive.
constexpr size_t DW_NOALLOC_BYTES = (size_t)1 << 20;
constexpr int DW_NOALLOC_MAX_DEVICES = 64;
static __device__ __align__(256) unsigned char dw_wg_scratch[DW_NOALLOC_BYTES];
static float *g_dw_wg_scratch_ptr[DW_NOALLOC_MAX_DEVICES] = {};

int dw_noalloc_setup(int device) {
    if (device < 0 || device >= DW_NOALLOC_MAX_DEVICES) return 0;  // such a device runs the allocating entry points only
    if (g_dw_wg_scratch_ptr[device]) return 0;
    void *ptr = nullptr;
    if (!hip_ok(hipGetSymbolAddress(&ptr, HIP_SYMBOL(dw_wg_scratch)), "hipGetSymbolAddress(dw_wg_scratch)")) return 2;
    g_dw_wg_scratch_ptr[device] = static_cast<float *>(ptr);
    return 0;
}

// `fixed` / `fixed_bytes`: partial sums go to this buffer instead of the growing workspace, tensors must already
// be in device memory, and the call fails rather than allocate (the allocation-free entry point).
template <typename T, typename Args>
static int dw_step(const Args *a, int ns, int step, int sh, int sw, const char *fn, float *fixed = nullptr,
                   size_t fixed_bytes = 0) {
    DwGeom g;
    if (int rc = dw_geom(a, g, sh, sw, fn)) return rc;
    if (ns <= 0) return 0;
    if (!fixed && !ensure_init()) return 2;
    State &st = state();
    bool too_big = false;
    auto partials = [&](size_t bytes) -> float * {
        if (!fixed) return workspace(bytes);
        if (bytes > fixed_bytes) {
            set_error("%s: the partial sums of this call take %zu bytes, the fixed buffer of the allocation-free "
                      "entry point holds %zu", fn, bytes, fixed_bytes);
            too_big = true;
            return nullptr;
        }
        return fixed;
    };
    size_t in_n = (size_t)ns * g.C * g.H * g.W, out_n = (size_t)ns * g.C * g.Ho * g.Wo;
    size_t w_n = (size_t)g.C * g.Hk * g.Wk;
    Stager sg(fixed != nullptr);
    int rc = 0;
    // row-walking kernels: unit stride, square 3x3 / 5x5 kernel, rows wide enough to fill a wave
    const bool rows_path = sh == 1 && sw == 1 && g.Hk == g.Wk && (g.Hk == 3 || g.Hk == 5) && g.Wo >= 32 && g.W >= 32;
    const long planes = (long)ns * g.C;
    // plane-resident kernels: the same geometry with planes of at most 40 KB and enough of them to fill the
    // chip; measured faster for 2-byte elements (forward, input gradient, weight gradient) and for the fp32
    // forward and input gradient
    const size_t in_img = (size_t)g.H * g.W * sizeof(T) + 32, out_img = (size_t)g.Ho * g.Wo * sizeof(T) + 32;
    const bool plane_path = rows_path && in_img <= 40 * 1024 && out_img <= 40 * 1024 && planes >= 2L * st.num_cu &&
                            planes < ((long)1 << 31) && st.gemm_path != 1;
    // a single sample: one workgroup per channel produces the weight gradient in one launch
    const bool wg_single = rows_path && ns == 1 && in_img <= 40 * 1024 && out_img <= 40 * 1024 && st.gemm_path != 1;
    if (step == STEP_FW) {
        const T *X = sg.in(reinterpret_cast<const T *>(a->input->data), in_n);
        const T *Wt = sg.in(reinterpret_cast<const T *>(a->coeff->data), w_n);
        T *Y = sg.out(reinterpret_cast<T *>(a->output->data), out_n);
        if (sg.failed()) return sg.rejected() ? 1 : 2;
        if (plane_path) {
            if (g.Hk == 3)
                launch_dw_plane<T, 3, false>(X, Wt, Y, g.C, g.H, g.W, g.Ho, g.Wo, g.Up, g.Lp, planes, st.stream);
            else
                launch_dw_plane<T, 5, false>(X, Wt, Y, g.C, g.H, g.W, g.Ho, g.Wo, g.Up, g.Lp, planes, st.stream);
        } else if (rows_path) {
            int rbs = (g.Ho + DW_RB - 1) / DW_RB, ccs = (g.Wo + 63) / 64;
            long waves = planes * rbs * ccs;
            dim3 grid((unsigned)((waves + 3) / 4));
            if (g.Hk == 3)
                hipLaunchKernelGGL((dw_rows_kernel<T, 3, false>), grid, dim3(256), 0, st.stream, X, Wt, Y, g.C, g.H,
                                   g.W, g.Ho, g.Wo, g.Up, g.Lp, rbs, ccs, waves);
            else
                hipLaunchKernelGGL((dw_rows_kernel<T, 5, false>), grid, dim3(256), 0, st.stream, X, Wt, Y, g.C, g.H,
                                   g.W, g.Ho, g.Wo, g.Up, g.Lp, rbs, ccs, waves);
        } else {
            hipLaunchKernelGGL((dw_fw_kernel<T>), dim3(nblocks(out_n)), dim3(256), 0, st.stream, X, Wt, Y, g, out_n);
        }
    } else if (step == STEP_IN_GRAD) {
        const T *dY = sg.in(reinterpret_cast<const T *>(a->output->diff), out_n);
        const T *Wt = sg.in(reinterpret_cast<const T *>(a->coeff->data), w_n);
        T *dX = sg.out(reinterpret_cast<T *>(a->input->diff), in_n);
        if (sg.failed()) return sg.rejected() ? 1 : 2;
        if (plane_path) {
            if (g.Hk == 3)
                launch_dw_plane<T, 3, true>(dY, Wt, dX, g.C, g.Ho, g.Wo, g.H, g.W, g.Hk - 1 - g.Up, g.Wk - 1 - g.Lp,
                                            planes, st.stream);
            else
                launch_dw_plane<T, 5, true>(dY, Wt, dX, g.C, g.Ho, g.Wo, g.H, g.W, g.Hk - 1 - g.Up, g.Wk - 1 - g.Lp,
                                            planes, st.stream);
        } else if (rows_path) {
            int rbs = (g.H + DW_RB - 1) / DW_RB, ccs = (g.W + 63) / 64;
            long waves = planes * rbs * ccs;
            dim3 grid((unsigned)((waves + 3) / 4));
            if (g.Hk == 3)
                hipLaunchKernelGGL((dw_rows_kernel<T, 3, true>), grid, dim3(256), 0, st.stream, dY, Wt, dX, g.C,
                                   g.Ho, g.Wo, g.H, g.W, g.Hk - 1 - g.Up, g.Wk - 1 - g.Lp, rbs, ccs, waves);
            else
                hipLaunchKernelGGL((dw_rows_kernel<T, 5, true>), grid, dim3(256), 0, st.stream, dY, Wt, dX, g.C,
                                   g.Ho, g.Wo, g.H, g.W, g.Hk - 1 - g.Up, g.Wk - 1 - g.Lp, rbs, ccs, waves);
        } else {
            hipLaunchKernelGGL((dw_ig_kernel<T>), dim3(nblocks(in_n)), dim3(256), 0, st.stream, dY, Wt, dX, g, in_n);
        }
    } else if (plane_path || wg_single) {
        const T *X = sg.in(reinterpret_cast<const T *>(a->input->data), in_n);
        const T *dY = sg.in(reinterpret_cast<const T *>(a->output->diff), out_n);
        T *dW = sg.out(reinterpret_cast<T *>(a->coeff->diff), w_n);
        if (sg.failed()) return sg.rejected() ? 1 : 2;
        const int taps = g.Hk * g.Wk;
        // sample groups: about four workgroups per CU
        int sgroups = (int)((4L * st.num_cu + g.C - 1) / g.C);
        if (sgroups > ns) sgroups = ns;
        if (sgroups < 1) sgroups = 1;
        const int per_group = (ns + sgroups - 1) / sgroups;
        sgroups = (ns + per_group - 1) / per_group;
        float *part = partials((size_t)sgroups * g.C * taps * sizeof(float));
        if (!part) return sg.finish(too_big ? 1 : 2);
        T *direct = sgroups == 1 ? dW : nullptr;  // one group: the kernel writes the gradient, no second launch
        const int x_vecs = (int)((in_img + 15) / 16);
        const size_t lds = (size_t)x_vecs * 16 + out_img;
        dim3 grid(g.C, sgroups);
        bool pairs = false;
        if constexpr (sizeof(T) == 2) {
            pairs = g.W % 2 == 0 && g.Wo % 2 == 0 && g.Lp % 2 == 0 && reinterpret_cast<uintptr_t>(X) % 4 == 0 &&
                    reinterpret_cast<uintptr_t>(dY) % 4 == 0;
            if (pairs && g.Hk == 3 && ns > 1) {
                hipLaunchKernelGGL(dw_wg_direct_kernel, grid, dim3(256), 0, st.stream, X, dY, part, g.C, ns, per_group, g.H,
                                   g.W, g.Ho, g.Wo, g.Up, g.Lp, direct);
            } else if (pairs) {
                if (g.Hk == 3)
                    hipLaunchKernelGGL((dw_wg_plane_pairs_kernel<3>), grid, dim3(256), lds, st.stream, X, dY, part, g.C,
                                       ns, per_group, g.H, g.W, g.Ho, g.Wo, g.Up, g.Lp, x_vecs, direct);
                else
                    hipLaunchKernelGGL((dw_wg_plane_pairs_kernel<5>), grid, dim3(256), lds, st.stream, X, dY, part, g.C,
                                       ns, per_group, g.H, g.W, g.Ho, g.Wo, g.Up, g.Lp, x_vecs, direct);
            }
        }
        if (pairs) {
        } else if (g.Hk == 3)
            hipLaunchKernelGGL((dw_wg_plane_kernel<T, 3>), grid, dim3(256), lds, st.stream, X, dY, part, g.C, ns,
                               per_group, g.H, g.W, g.Ho, g.Wo, g.Up, g.Lp, x_vecs, direct);
        else
            hipLaunchKernelGGL((dw_wg_plane_kernel<T, 5>), grid, dim3(256), lds, st.stream, X, dY, part, g.C, ns,
                               per_group, g.H, g.W, g.Ho, g.Wo, g.Up, g.Lp, x_vecs, direct);
        if (!direct)
            hipLaunchKernelGGL((dw_wg_reduce_kernel2<T>), dim3(g.C), dim3(256), 0, st.stream, part, dW, sgroups, g.C, 1,
                               taps);
    } else if (rows_path) {
        const T *X = sg.in(reinterpret_cast<const T *>(a->input->data), in_n);
        const T *dY = sg.in(reinterpret_cast<const T *>(a->output->diff), out_n);
        T *dW = sg.out(reinterpret_cast<T *>(a->coeff->diff), w_n);
        if (sg.failed()) return sg.rejected() ? 1 : 2;
        // strips of rows: enough waves to fill the chip, at least 8 rows each
        int ccs = (g.Wo + 63) / 64;
        long want = 8L * st.num_cu * 4;
        int rbs = (int)((want + planes * ccs - 1) / (planes * ccs));
        if (rbs > (g.Ho + 7) / 8) rbs = (g.Ho + 7) / 8;
        if (rbs < 1) rbs = 1;
        int rows_per = (g.Ho + rbs - 1) / rbs;
        rbs = (g.Ho + rows_per - 1) / rows_per;
        long waves = planes * rbs * ccs;
        int taps = g.Hk * g.Wk;
        float *part = partials((size_t)waves * taps * sizeof(float));
        if (!part) return sg.finish(too_big ? 1 : 2);
        dim3 grid((unsigned)((waves + 3) / 4));
        if (g.Hk == 3)
            hipLaunchKernelGGL((dw_wg_rows_kernel<T, 3>), grid, dim3(256), 0, st.stream, X, dY, part, g.C, g.H, g.W,
                               g.Ho, g.Wo, g.Up, g.Lp, rbs, ccs, rows_per, waves);
        else
            hipLaunchKernelGGL((dw_wg_rows_kernel<T, 5>), grid, dim3(256), 0, st.stream, X, dY, part, g.C, g.H, g.W,
                               g.Ho, g.Wo, g.Up, g.Lp, rbs, ccs, rows_per, waves);
        hipLaunchKernelGGL((dw_wg_reduce_kernel2<T>), dim3(g.C), dim3(256), 0, st.stream, part, dW, ns, g.C,
                           rbs * ccs, taps);
    } else {
        const T *X = sg.in(reinterpret_cast<const T *>(a->input->data), in_n);
        const T *dY = sg.in(reinterpret_cast<const T *>(a->output->diff), out_n);
        T *dW = sg.out(reinterpret_cast<T *>(a->coeff->diff), w_n);
        if (sg.failed()) return sg.rejected() ? 1 : 2;
        size_t n = (size_t)ns * g.Ho * g.Wo;
        // enough chunks for a few workgroups per CU, at least 1024 pixels each
        int chunks = (int)((4 * (size_t)st.num_cu + g.C - 1) / g.C);
        size_t maxc = (n + 1023) / 1024;
        if ((size_t)chunks > maxc) chunks = (int)maxc;
        if (chunks < 1) chunks = 1;
        int per = (int)((n + chunks - 1) / chunks);
        chunks = (int)((n + per - 1) / per);
        float *part = partials((size_t)chunks * w_n * sizeof(float));
        if (!part) return sg.finish(too_big ? 1 : 2);
        int taps = g.Hk * g.Wk;
        dim3 grid(g.C, chunks);
        if (taps <= 9)
            hipLaunchKernelGGL((dw_wg_kernel<T, 9>), grid, dim3(256), 0, st.stream, X, dY, part, g, ns, per);
        else if (taps <= 25)
            hipLaunchKernelGGL((dw_wg_kernel<T, 25>), grid, dim3(256), 0, st.stream, X, dY, part, g, ns, per);
        else
            hipLaunchKernelGGL((dw_wg_kernel<T, 49>), grid, dim3(256), 0, st.stream, X, dY, part, g, ns, per);
        hipLaunchKernelGGL((dw_wg_reduce_kernel<T>), dim3(nblocks(w_n)), dim3(256), 0, st.stream, part, dW,
                           (int)w_n, chunks);
    }
    if (!hip_ok(hipGetLastError(), "depthwise launch")) rc = 2;
    return sg.finish(rc);
}

// ---- Patch-matrix builders (index work) -------------------------------------------------
struct PatchGeom {
    int C;       // channels of the source tensor (Cin for mod 0, Cout for mod 1)
    int Hs, Ws;  // source extent
    int Hp, Wp;  // patch grid extent (output pixels for mod 0, input pixels for mod 1)
    int Hk, Wk;
    int h_mul, h_add, w_mul, w_add;  // source row = hp*h_mul + h_add + hk
    int hwc;
    int col_major;  // 0: buf[p*Q + q] (im2row); 1: buf[q*P + p] (im2col)
};

typedef unsigned PatchPiece __attribute__((ext_vector_type(4)));  // (a built-in vector: loads from any address space)
__device__ const PatchPiece patch_zero = {0u, 0u, 0u, 0u};  // what the window holds outside the tensor

// buf(p, q) = src[c, hp*h_mul + h_add + hk, wp*w_mul + w_add + wk] or 0 outside,
// p = hp*Wp + wp, q = (c,hk,wk) for CHW and (hk,wk,c) for HWC.
// A thread writes PER consecutive elements of the buffer (one 16-byte store when PER elements fill 16 bytes and
// the buffer is aligned): its first index is decoded with divisions once, the following ones by carrying
// (wk -> hk -> c -> next row, or wp -> hp -> next column), so the index arithmetic is a handful of additions
// per element and the write side - nine times the bytes of the read side for a 3x3 filter - moves whole chunks.
template <typename T, int PER>
__global__ __launch_bounds__(256) void patch_kernel(const T *__restrict__ src, T *__restrict__ buf, PatchGeom g,
                                                    size_t total) {
    // (the host keeps the matrix below 2^32 elements: 32-bit index arithmetic)
    const size_t idx0 = ((size_t)blockIdx.x * 256 + threadIdx.x) * PER;
    if (idx0 >= total) return;
    const unsigned Q = (unsigned)(g.C * g.Hk * g.Wk), P = (unsigned)(g.Hp * g.Wp), i32 = (unsigned)idx0;
    unsigned p, q;
    if (!g.col_major) {
        p = i32 / Q;
        q = i32 - p * Q;
    } else {
        q = i32 / P;
        p = i32 - q * P;
    }
    int hp = (int)(p / (unsigned)g.Wp), wp = (int)(p - (unsigned)hp * g.Wp);
    int c, hk, wk;
    if (!g.hwc) {
        const unsigned t = q / (unsigned)g.Wk;
        wk = (int)(q - t * g.Wk);
        c = (int)(t / (unsigned)g.Hk);
        hk = (int)(t - (unsigned)c * g.Hk);
    } else {
        const unsigned t = q / (unsigned)g.C;
        c = (int)(q - t * g.C);
        hk = (int)(t / (unsigned)g.Wk);
        wk = (int)(t - (unsigned)hk * g.Wk);
    }
    T v[PER];
#pragma unroll
    for (int e = 0; e < PER; ++e) {
        const int h = hp * g.h_mul + g.h_add + hk, w = wp * g.w_mul + g.w_add + wk;
        // (every lane always loads, what lies outside the tensor from a word of zeros: a load under a condition
        // becomes a branch with a wait of its own, one trip to memory per element; 32-bit offsets - the host keeps
        // the source below 2^32 elements)
        const bool ok = idx0 + e < total && (unsigned)h < (unsigned)g.Hs && (unsigned)w < (unsigned)g.Ws;
        const unsigned off = g.hwc ? ((unsigned)h * g.Ws + w) * g.C + c : ((unsigned)c * g.Hs + h) * g.Ws + w;
        typedef const T __attribute__((address_space(1))) *GlobalT;
        v[e] = *(ok ? (GlobalT)(src + off) : (GlobalT)&patch_zero);
        // next element of the buffer
        bool next_q = true, next_p = false;
        if (g.col_major) {  // p runs fastest
            next_q = false;
            next_p = true;
        }
        if (next_q) {
            if (!g.hwc) {
                if (++wk == g.Wk) {
                    wk = 0;
                    if (++hk == g.Hk) {
                        hk = 0;
                        if (++c == g.C) {
                            c = 0;
                            next_p = true;
                        }
                    }
                }
            } else {
                if (++c == g.C) {
                    c = 0;
                    if (++wk == g.Wk) {
                        wk = 0;
                        if (++hk == g.Hk) {
                            hk = 0;
                            next_p = true;
                        }
                    }
                }
            }
        }
        if (next_p) {
            if (++wp == g.Wp) {
                wp = 0;
                if (++hp == g.Hp) {
                    hp = 0;
                    if (g.col_major) {  // the column is complete: on to the next q
                        if (!g.hwc) {
                            if (++wk == g.Wk) {
                                wk = 0;
                                if (++hk == g.Hk) {
                                    hk = 0;
                                    ++c;
                                }
                            }
                        } else {
                            if (++c == g.C) {
                                c = 0;
                                if (++wk == g.Wk) {
                                    wk = 0;
                                    ++hk;
                                }
                            }
                        }
                    }
                }
            }
        }
    }
    if (PER * sizeof(T) == 16 && idx0 + PER <= total) {
        union {
            uint4 u;
            T e[PER];
        } pack;
#pragma unroll
        for (int e = 0; e < PER; ++e) pack.e[e] = v[e];
        *reinterpret_cast<uint4 *>(buf + idx0) = pack.u;
    } else {
#pragma unroll
        for (int e = 0; e < PER; ++e)
            if (idx0 + e < total) buf[idx0 + e] = v[e];
    }
}

// Row-major patch matrix of a channel-major tensor (im2row, the layout the reference's layers use) through LDS:
// a workgroup owns R consecutive patch-grid positions of one grid row and CB channels.  It stages the source
// window those patches cover ([CB][Hk][(R-1)*w_mul + Wk] elements, zero outside the tensor) with coalesced reads -
// every source element is fetched once per workgroup instead of once per tap - and then writes its part of the
// R buffer rows as 16-byte chunks, each gathered from LDS.  Divisions by the runtime extents are multiplications
// by ceil(2^32 / d) (exact for dividends below 2^16).
// A vector memory instruction occupies the address unit for its 64 lanes whatever each lane moves, so the window
// is read in as few instructions as the layout allows: WIDE (rows of the tensor start on 16-byte boundaries) takes
// the aligned 16-byte pieces that cover the window - the window then starts up to a piece early, `shift` elements
// that the offsets table skips - and otherwise one element per lane, one wave per window row.

template <typename T, bool WIDE>
__global__ __launch_bounds__(256) void patch_rows_kernel(const T *__restrict__ src, T *__restrict__ buf, PatchGeom g, int R,
                                                         int CB, int LW, unsigned m_pk, unsigned m_wk, unsigned m_hk) {
    constexpr int VEC = 16 / (int)sizeof(T);
    // (as global-memory pointers: a generic one would load through the flat path, whose waits are shared with LDS)
    typedef const T __attribute__((address_space(1))) *GlobalT;
    typedef const PatchPiece __attribute__((address_space(1))) *GlobalPiece;
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const int PK = g.Hk * g.Wk, Q = g.C * PK, nq = CB * PK;
    unsigned short *offs = reinterpret_cast<unsigned short *>(smem);                    // [nq], nq a multiple of VEC
    T *lds = reinterpret_cast<T *>(smem + (((size_t)nq * 2 + 15) & ~(size_t)15));      // [CB * Hk][LW], one spare slot
    const int wp0 = blockIdx.x * R, hp = blockIdx.y, c0 = blockIdx.z * CB;
    const int nr = min(R, g.Wp - wp0);
    const int w_first = wp0 * g.w_mul + g.w_add, h_first = hp * g.h_mul + g.h_add;
    const int w_start = WIDE ? (w_first & ~(VEC - 1)) : w_first, shift = w_first - w_start;  // (& rounds down below 0 too)
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    // where column q = (channel, filter row, filter column) of a buffer row starts in the staged window
    for (int q = threadIdx.x; q < nq; q += 256) {
        const unsigned c_l = div_magic((unsigned)q, m_pk), t = (unsigned)q - c_l * PK;
        const unsigned hk = div_magic(t, m_wk), wk = t - hk * g.Wk;
        offs[q] = (unsigned short)((c_l * g.Hk + hk) * LW + wk + shift);
    }
    const int rows = CB * g.Hk, width = (R - 1) * g.w_mul + g.Wk;  // the window: rows, and what the patches reach of one
    // Every lane always loads and always stores: a load under a condition becomes a branch with a wait of its own,
    // and the compiler moves a load into the branch that holds its only use.  What lies outside the tensor is read
    // from a piece of zeros; what lies outside the window is written to the spare slot behind it.
    if (WIDE) {
        const int np = (shift + width + VEC - 1) / VEC, items = rows * np;  // pieces per row; LW holds np whole pieces
        const unsigned m_np = (unsigned)((((unsigned long long)1 << 32) + np - 1) / np);
        for (int i0 = threadIdx.x; i0 < items; i0 += 4 * 256) {
            PatchPiece v[4];
            int at[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int item = i0 + u * 256;
                const int r = (int)div_magic((unsigned)min(item, items - 1), m_np), piece = min(item, items - 1) - r * np;
                const int c_l = (int)div_magic((unsigned)r, m_hk), h = h_first + (r - c_l * g.Hk), w = w_start + piece * VEC;
                const bool ok = (unsigned)h < (unsigned)g.Hs && (unsigned)w < (unsigned)g.Ws;  // (a piece is all in or all out)
                const int off = ((c0 + c_l) * g.Hs + h) * g.Ws + w;  // (below 2^31: the host checks the tensor's size)
                v[u] = *(ok ? (GlobalPiece)(src + off) : (GlobalPiece)&patch_zero);
                at[u] = item < items ? r * LW + piece * VEC : rows * LW;
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {  // (rows start on 4-byte boundaries only: their pitch is an odd number of dwords)
                unsigned *dst = reinterpret_cast<unsigned *>(lds + at[u]);
                dst[0] = v[u].x; dst[1] = v[u].y; dst[2] = v[u].z; dst[3] = v[u].w;
            }
        }
    } else {
        const int w_lane = w_first + lane;
        const bool col_ok = (unsigned)w_lane < (unsigned)g.Ws && lane < width;
        for (int r0 = wave; r0 < rows; r0 += 64) {
            T v[16];
#pragma unroll
            for (int u = 0; u < 16; ++u) {
                const int r = min(r0 + 4 * u, rows - 1);
                const int c_l = (int)div_magic((unsigned)r, m_hk), h = h_first + (r - c_l * g.Hk);
                const bool ok = (unsigned)h < (unsigned)g.Hs && col_ok;
                const int off = ((c0 + c_l) * g.Hs + h) * g.Ws + w_lane;
                v[u] = *(ok ? (GlobalT)(src + off) : (GlobalT)&patch_zero);
            }
#pragma unroll
            for (int u = 0; u < 16; ++u) lds[lane < width && r0 + 4 * u < rows ? (r0 + 4 * u) * LW + lane : rows * LW] = v[u];
        }
    }
    __syncthreads();
    // a thread keeps one chunk position of the buffer rows (its table entries stay in registers) and walks down the
    // positions; a row piece longer than the workgroup takes several sweeps
    const int cpr = nq / VEC;  // chunks of this workgroup per buffer row
    const int span = min(cpr, 256), pstep = 256 / span, p0 = threadIdx.x / span;
    T *base = buf + ((size_t)hp * g.Wp + wp0) * Q + (size_t)c0 * PK;
    for (int qc = threadIdx.x - p0 * span; qc < cpr && p0 < pstep; qc += span) {
        int o[VEC];
        if (VEC == 8) {
            const uint4 t4 = *reinterpret_cast<const uint4 *>(offs + qc * 8);
            o[0] = t4.x & 0xffffu; o[1] = t4.x >> 16; o[2] = t4.y & 0xffffu; o[3] = t4.y >> 16;
            o[4 % VEC] = t4.z & 0xffffu; o[5 % VEC] = t4.z >> 16; o[6 % VEC] = t4.w & 0xffffu; o[7 % VEC] = t4.w >> 16;
        } else {
            const uint2 t2 = *reinterpret_cast<const uint2 *>(offs + qc * 4);
            o[0] = t2.x & 0xffffu; o[1] = t2.x >> 16; o[2] = t2.y & 0xffffu; o[3] = t2.y >> 16;
        }
        const T *win = lds + p0 * g.w_mul;
        T *dst = base + (size_t)p0 * Q + qc * VEC;
        for (int p_l = p0; p_l < nr; p_l += pstep) {
            union {
                uint4 u;
                T e[VEC];
            } v;
#pragma unroll
            for (int e = 0; e < VEC; ++e) v.e[e] = win[o[e]];
            *reinterpret_cast<uint4 *>(dst) = v.u;
            win += pstep * g.w_mul;
            dst += (size_t)pstep * Q;
        }
    }
}

// Column-major patch matrix (im2col) of a channel-major tensor at unit column stride: row q = (c, hk, wk) of the
// buffer is channel c's plane shifted by the tap, so a 16-byte chunk of it (consecutive grid columns of one grid
// row, when the grid's width is a whole number of chunks) is one run of consecutive source elements.  A thread
// loads that run with one 16-byte access at element alignment - from a start moved inside the row where the run
// would begin before it or end behind it - and shifts the 128 bits by the distance moved, which leaves zeros in
// exactly the positions that lie outside the row; a run in a row outside the tensor reads a piece of zeros.  One
// division per workgroup, reciprocal multiplications on the small per-thread rests.
struct PatchCols {
    int cpr, wpc;              // chunks per buffer row, chunks per grid row
    unsigned m_cpr, m_wpc, m_pk, m_wk;
};

template <typename T>
__global__ __launch_bounds__(256) void patch_cols_kernel(const T *__restrict__ src, T *__restrict__ buf, PatchGeom g,
                                                         PatchCols k, unsigned chunks) {
    constexpr int VEC = 16 / (int)sizeof(T), EB = 8 * (int)sizeof(T);
    typedef unsigned Run __attribute__((ext_vector_type(4), aligned(2)));  // (element alignment of the narrower type)
    typedef const Run __attribute__((address_space(1))) *GlobalRun;
    const unsigned B = blockIdx.x * 256u, i = B + threadIdx.x;
    if (i >= chunks) return;
    const int PK = g.Hk * g.Wk;
    const unsigned q_B = B / (unsigned)k.cpr, r_B = B - q_B * k.cpr;
    const unsigned c_B = q_B / (unsigned)PK, t_B = q_B - c_B * PK;
    const unsigned x = r_B + threadIdx.x, dq = div_magic(x, k.m_cpr), r = x - dq * k.cpr;
    const unsigned t2 = t_B + dq, dc = div_magic(t2, k.m_pk), t3 = t2 - dc * PK;
    const int c = (int)(c_B + dc), hk = (int)div_magic(t3, k.m_wk), wk = (int)t3 - hk * g.Wk;
    const int hp = (int)div_magic(r, k.m_wpc), wp0 = ((int)r - hp * k.wpc) * VEC;
    const int h = hp * g.h_mul + g.h_add + hk, w0 = wp0 + g.w_add + wk;
    const int w_in = min(max(w0, 0), g.Ws - VEC), d = w0 - w_in;  // d > 0: the run ends behind the row
    const bool ok = (unsigned)h < (unsigned)g.Hs && d > -VEC && d < VEC;
    const unsigned off = ((unsigned)c * g.Hs + h) * g.Ws + w_in;
    Run v = *(ok ? (GlobalRun)(src + off) : (GlobalRun)&patch_zero);
    const int bits = (d < 0 ? -d : d) * EB;
    if (d > 0) {  // towards element 0
        if (bits & 64) v = Run{v.z, v.w, 0u, 0u};
        if (bits & 32) v = Run{v.y, v.z, v.w, 0u};
        const unsigned bs = bits & 31;
        v = Run{__builtin_amdgcn_alignbit(v.y, v.x, bs), __builtin_amdgcn_alignbit(v.z, v.y, bs),
                __builtin_amdgcn_alignbit(v.w, v.z, bs), v.w >> bs};
    } else if (d < 0) {
        if (bits & 64) v = Run{0u, 0u, v.x, v.y};
        if (bits & 32) v = Run{0u, v.x, v.y, v.z};
        const unsigned bs = bits & 31;  // (0 or 16: a left shift by 16 is alignbit(hi, lo, 16) one dword up)
        if (bs) v = Run{v.x << 16, __builtin_amdgcn_alignbit(v.y, v.x, 16), __builtin_amdgcn_alignbit(v.z, v.y, 16),
                        __builtin_amdgcn_alignbit(v.w, v.z, 16)};
    }
    typedef unsigned Chunk __attribute__((ext_vector_type(4)));
    *reinterpret_cast<Chunk *>(buf + (size_t)i * VEC) = Chunk{v.x, v.y, v.z, v.w};
}

// The column-major patch matrix at unit strides from the source's side: a row (c, hk, wk) of the matrix is the image
// plane c shifted by (hk - pad, wk - pad), so one 16-byte piece of a source row - with its left and right neighbours -
// is all that the K x K pieces at the same place of the K x K shifted copies need.  A thread loads the three aligned
// pieces once (zeros outside the tensor) and stores K x K pieces: elements VEC + d .. 2 VEC + d - 1 of the three
// pieces in a row, d = wk - PADL, cut out with compile-time dword selections and 16-bit funnel shifts.  Source rows
// run from -padU to Hp + K - 2 - padU, so that the matrix rows over the padding are written too.  The write side moves
// as in a fill kernel and the read side is a ninth of it.
template <typename T, int K, int PADL>
__global__ __launch_bounds__(256) void patch_cols_shifted_kernel(const T *__restrict__ src, T *__restrict__ buf,
                                                                 PatchGeom g, int wpcs, unsigned m_wpcs, int pieces) {
    constexpr int VEC = 16 / (int)sizeof(T), EPD = 4 / (int)sizeof(T);  // elements per piece, per dword
    typedef const PatchPiece __attribute__((address_space(1))) *GlobalPiece;
    const int i = blockIdx.x * 256 + threadIdx.x, c = blockIdx.y;
    if (i >= pieces) return;
    const int hv = (int)div_magic((unsigned)i, m_wpcs), wpc = i - hv * wpcs;
    const int h = hv + g.h_add;  // (h_add = -padU)
    const bool row_ok = (unsigned)h < (unsigned)g.Hs;
    const unsigned off = ((unsigned)c * g.Hs + (row_ok ? h : 0)) * g.Ws + wpc * VEC;
    const bool l_ok = row_ok && wpc > 0, r_ok = row_ok && (wpc + 2) * VEC <= g.Ws;
    const PatchPiece mine = *(row_ok ? (GlobalPiece)(src + off) : (GlobalPiece)&patch_zero);
    const PatchPiece left = *(l_ok ? (GlobalPiece)(src + off - VEC) : (GlobalPiece)&patch_zero);
    const PatchPiece right = *(r_ok ? (GlobalPiece)(src + off + VEC) : (GlobalPiece)&patch_zero);
    const unsigned win[12] = {left.x, left.y, left.z, left.w, mine.x, mine.y, mine.z, mine.w, right.x, right.y, right.z, right.w};
    PatchPiece out[K];
#pragma unroll
    for (int wk = 0; wk < K; ++wk) {
        const int s0 = VEC + wk - PADL, dw = s0 / EPD, sub = s0 % EPD;  // (compile-time after unrolling)
        if (sub == 0)
            out[wk] = PatchPiece{win[dw], win[dw + 1], win[dw + 2], win[dw + 3]};
        else
            out[wk] = PatchPiece{__builtin_amdgcn_alignbit(win[dw + 1], win[dw], 16), __builtin_amdgcn_alignbit(win[dw + 2], win[dw + 1], 16),
                                 __builtin_amdgcn_alignbit(win[dw + 3], win[dw + 2], 16), __builtin_amdgcn_alignbit(win[dw + 4], win[dw + 3], 16)};
    }
    const size_t P = (size_t)g.Hp * g.Wp;
#pragma unroll
    for (int hk = 0; hk < K; ++hk) {
        const int hp = hv - hk;
        if ((unsigned)hp < (unsigned)g.Hp) {
            T *row = buf + ((size_t)(c * K + hk) * K) * P + (size_t)hp * g.Wp + wpc * VEC;
#pragma unroll
            for (int wk = 0; wk < K; ++wk) *reinterpret_cast<PatchPiece *>(row + wk * P) = out[wk];
        }
    }
}

template <typename T, int K, int PADL>
static int launch_patch_cols_shifted(const T *src, T *buf, const PatchGeom &g) {
    constexpr int VEC = 16 / (int)sizeof(T);
    const int wpcs = g.Wp / VEC, pieces = (g.Hp + K - 1) * wpcs;
    const unsigned m = (unsigned)((((unsigned long long)1 << 32) + wpcs - 1) / wpcs);
    hipLaunchKernelGGL((patch_cols_shifted_kernel<T, K, PADL>), dim3((pieces + 255) / 256, g.C), dim3(256), 0, state().stream,
                       src, buf, g, wpcs, wpcs == 1 ? 0u : m, pieces);
    return hip_ok(hipGetLastError(), "patch launch") ? 0 : 2;
}

// 0 = launched; -1 = the geometry does not fit.
template <typename T>
static int patch_cols_shifted(const T *src, T *buf, const PatchGeom &g) {
    constexpr int VEC = 16 / (int)sizeof(T);
    if (g.hwc || !g.col_major || g.w_mul != 1 || g.h_mul != 1 || g.Hk != g.Wk || g.Wp % VEC || g.Ws % VEC || g.Wp > g.Ws ||
        g.C > 65535 || reinterpret_cast<uintptr_t>(buf) % 16 || reinterpret_cast<uintptr_t>(src) % 16)
        return -1;
    // (32-bit element offsets into the source, quotients by multiplication below 2^16 pieces per plane)
    if ((long long)g.C * g.Hs * g.Ws >= ((long long)1 << 31) || (long long)(g.Hp + g.Hk) * (g.Wp / VEC) >= 65536) return -1;
    const int K = g.Hk, padl = -g.w_add;
    if (K == 3 && padl == 1) return launch_patch_cols_shifted<T, 3, 1>(src, buf, g);
    if (K == 3 && padl == 0) return launch_patch_cols_shifted<T, 3, 0>(src, buf, g);
    if (K == 5 && padl == 2) return launch_patch_cols_shifted<T, 5, 2>(src, buf, g);
    if (K == 7 && padl == 3) return launch_patch_cols_shifted<T, 7, 3>(src, buf, g);
    return -1;
}

// 0 = launched; -1 = the geometry does not fit (the caller takes the general kernel).
template <typename T>
static int patch_cols(const T *src, T *buf, const PatchGeom &g) {
    constexpr int VEC = 16 / (int)sizeof(T);
    if (g.hwc || !g.col_major || g.w_mul != 1 || g.Wp % VEC || g.Ws < VEC || reinterpret_cast<uintptr_t>(buf) % 16)
        return -1;
    const long long P = (long long)g.Hp * g.Wp, PK = (long long)g.Hk * g.Wk, chunks = P / VEC * PK * g.C;
    // (the reciprocal divisions are exact below 2^16: a row or tap index at most a workgroup's 256 chunks further on)
    if (P / VEC + 256 >= 65536 || PK + 256 >= 65536 || chunks >= ((long long)1 << 32) / 256 * 256) return -1;
    auto magic = [](unsigned d) { return (unsigned)((((unsigned long long)1 << 32) + d - 1) / d); };
    PatchCols k;
    k.cpr = (int)(P / VEC);
    k.wpc = g.Wp / VEC;
    k.m_cpr = magic(k.cpr); k.m_wpc = magic(k.wpc); k.m_pk = magic((unsigned)PK); k.m_wk = magic(g.Wk);
    hipLaunchKernelGGL((patch_cols_kernel<T>), dim3((unsigned)((chunks + 255) / 256)), dim3(256), 0, state().stream, src, buf, g,
                       k, (unsigned)chunks);
    return hip_ok(hipGetLastError(), "patch launch") ? 0 : 2;
}

// 0 = launched; -1 = the geometry does not fit (the caller takes the general kernel).
template <typename T>
static int patch_rows(const T *src, T *buf, const PatchGeom &g) {
    constexpr int VEC = 16 / (int)sizeof(T), ES = (int)sizeof(T);
    if (g.hwc || g.col_major) return -1;
    const int PK = g.Hk * g.Wk;
    const long long Q = (long long)g.C * PK;
    if (reinterpret_cast<uintptr_t>(buf) % 16 || (Q * ES) % 16 || g.Wp < 16 || Q >= 65536 || g.Hp >= 65536 || g.Wk > 32 ||
        g.w_mul > 8 || (long long)(g.C + 64) * g.Hs * g.Ws >= ((long long)1 << 31))  // (32-bit element offsets, with slack)
        return -1;
    // rows of the tensor that start on 16-byte boundaries are read as aligned 16-byte pieces
    const bool wide = ((size_t)g.Ws * ES) % 16 == 0 && reinterpret_cast<uintptr_t>(src) % 16 == 0;
    // positions per workgroup: a window row of at most 64 elements (one pass of a wave) - half that with pieces,
    // whose loads are few either way: more and shorter workgroups overlap their load and store phases better -
    // and then the same number for every workgroup of a grid row
    int R = (64 - g.Wk) / g.w_mul + 1;
    if (wide && R >= 32) R = (R + 1) / 2;
    if (R > g.Wp) R = g.Wp;
    R = (g.Wp + (g.Wp + R - 1) / R - 1) / ((g.Wp + R - 1) / R);
    // row pitch of the window: an odd number of dwords, so that the rows the lanes of a wave gather from (every
    // Hk-th one for neighbouring channels) spread over the LDS banks; with pieces, room for the whole pieces that
    // cover a window starting anywhere in its first piece
    int LW = (R - 1) * g.w_mul + g.Wk;
    if (wide) LW = (VEC - 1 + LW + VEC - 1) / VEC * VEC;
    LW = ES == 2 ? (((LW + 1) & ~1) | 2) : (LW | 1);
    // (table of column offsets, window, one spare slot)
    auto bytes = [&](int cb) { return (((size_t)cb * PK * 2 + 15) & ~(size_t)15) + (size_t)cb * g.Hk * LW * ES + 16; };
    int CB = g.C;
    while (bytes(CB) > 40 * 1024 && CB % 2 == 0) CB /= 2;
    // whole buffer rows per workgroup (one contiguous run of R x Q elements) unless that leaves CUs idle; a
    // workgroup's piece of a buffer row stays a few cache lines long
    const long long per_z = (long long)((g.Wp + R - 1) / R) * g.Hp;
    while (per_z * (g.C / CB) < 2LL * state().num_cu && CB % 2 == 0 && (CB / 2) * PK * ES >= 256 && ((CB / 2) * PK) % VEC == 0)
        CB /= 2;
    if (bytes(CB) > 64 * 1024 || (CB * PK) % VEC || CB * g.Hk * LW >= 65536 || g.C / CB >= 65536) return -1;
    auto magic = [](unsigned d) { return (unsigned)((((unsigned long long)1 << 32) + d - 1) / d); };
    dim3 grid((g.Wp + R - 1) / R, g.Hp, g.C / CB);
    if (wide)
        hipLaunchKernelGGL((patch_rows_kernel<T, true>), grid, dim3(256), bytes(CB), state().stream, src, buf, g, R, CB, LW,
                           magic(PK), magic(g.Wk), magic(g.Hk));
    else
        hipLaunchKernelGGL((patch_rows_kernel<T, false>), grid, dim3(256), bytes(CB), state().stream, src, buf, g, R, CB,
                           LW, magic(PK), magic(g.Wk), magic(g.Hk));
    return hip_ok(hipGetLastError(), "patch launch") ? 0 : 2;
}

template <typename T, typename Args>
static int patch_build(const Args *a, int col_major, const char *fn) {
    if (!a || !a->input || !a->c || !a->output || !a->pBuffer) {
        printf("[%s] null argument structure\n", fn);
        set_error("%s: null argument structure", fn);
        return 1;
    }
    // the reference narrows these fields to 8 bits (lib/sources/pulp_im2col_fp32.c:39-48)
    const int Lp = (uint8_t)a->Lpad, Rp = (uint8_t)a->Rpad, Up = (uint8_t)a->Upad, Dp = (uint8_t)a->Dpad;
    const int mod = (uint8_t)a->mod, sh = (uint8_t)a->stride_h, sw = (uint8_t)a->stride_w, hwc = (uint8_t)a->HWC;
    const int Hin = a->input->H, Win = a->input->W, Cin = a->input->C;
    const int Hk = a->c->H, Wk = a->c->W, Co = a->output->C;
    if (hwc != 0 && hwc != 1) {
        printf("[%s:] Invalid HWC parameter (not 0 or 1)\n", fn);
        set_error("%s: HWC must be 0 or 1", fn);
        return 1;
    }
    if (Hin <= 0 || Win <= 0 || Cin <= 0 || Hk <= 0 || Wk <= 0) {
        printf("[%s] invalid tensor geometry\n", fn);
        set_error("%s: invalid tensor geometry", fn);
        return 1;
    }
    PatchGeom g = {};
    g.Hk = Hk;
    g.Wk = Wk;
    g.hwc = hwc;
    g.col_major = col_major;
    const T *src;
    size_t src_n;
    if (mod == 0) {
        if (sh == 0 || sw == 0 || Hin - Hk + Up + Dp < 0 || Win - Wk + Lp + Rp < 0) {
            printf("[%s] invalid stride or kernel size\n", fn);
            set_error("%s: invalid stride or kernel size", fn);
            return 1;
        }
        if ((Hin - Hk + Up + Dp + sh) % sh > 0) {
            printf("\n[%s] Invalid H stride (non multiple H sizes): have H_in=%d, H_ker=%d, U_pad=%d, D_pad=%d, "
                   "H_stride=%d, remainder=%d",
                   fn, Hin, Hk, Up, Dp, sh, (Hin - Hk + Up + Dp + sh) % sh);
            set_error("%s: H stride does not divide the padded extent", fn);
            return 1;
        }
        if ((Win - Wk + Lp + Rp + sw) % sw > 0) {
            printf("\n[%s] Invalid W stride (non multiple W sizes): have W_in=%d, W_ker=%d, L_pad=%d, R_pad=%d, "
                   "W_stride=%d, remainder=%d",
                   fn, Win, Wk, Lp, Rp, sw, (Win - Wk + Lp + Rp + sw) % sw);
            set_error("%s: W stride does not divide the padded extent", fn);
            return 1;
        }
        g.C = Cin;
        g.Hs = Hin;
        g.Ws = Win;
        g.Hp = (Hin - Hk + Up + Dp + sh) / sh;
        g.Wp = (Win - Wk + Lp + Rp + sw) / sw;
        g.h_mul = sh;
        g.h_add = -Up;
        g.w_mul = sw;
        g.w_add = -Lp;
        src = reinterpret_cast<const T *>(a->input->data);
        src_n = (size_t)Cin * Hin * Win;
    } else {
        // output-gradient patches with full (kernel-1) padding, unit stride
        g.C = Co;
        g.Hs = a->output->H;
        g.Ws = a->output->W;
        g.Hp = Hin;
        g.Wp = Win;
        g.h_mul = 1;
        g.h_add = -(Hk - 1);
        g.w_mul = 1;
        g.w_add = -(Wk - 1);
        src = reinterpret_cast<const T *>(a->output->diff);
        src_n = (size_t)Co * g.Hs * g.Ws;
    }
    if (!ensure_init()) return 2;
    size_t total = (size_t)g.Hp * g.Wp * g.C * Hk * Wk;
    Stager sg;
    const T *dsrc = sg.in(src, src_n);
    T *dbuf = sg.out(reinterpret_cast<T *>(a->pBuffer), total);
    if (sg.failed()) return 2;
    constexpr int VEC = 16 / (int)sizeof(T);
    if (total >= ((size_t)1 << 32) || src_n >= ((size_t)1 << 32)) {
        set_error("%s: patch matrix or source of 2^32 elements or more", fn);
        return sg.finish(1);
    }
    if (int rc = patch_rows<T>(dsrc, dbuf, g); rc >= 0) return sg.finish(rc);
    if (int rc = patch_cols_shifted<T>(dsrc, dbuf, g); rc >= 0) return sg.finish(rc);
    if (int rc = patch_cols<T>(dsrc, dbuf, g); rc >= 0) return sg.finish(rc);
    if (reinterpret_cast<uintptr_t>(dbuf) % 16 == 0)
        hipLaunchKernelGGL((patch_kernel<T, VEC>), dim3(nblocks((total + VEC - 1) / VEC)), dim3(256), 0, state().stream,
                           dsrc, dbuf, g, total);
    else
        hipLaunchKernelGGL((patch_kernel<T, 1>), dim3(nblocks(total)), dim3(256), 0, state().stream, dsrc, dbuf, g,
                           total);
    return sg.finish(hip_ok(hipGetLastError(), "patch launch") ? 0 : 2);
}

// bt[ci][co][i] = w[co][ci][P-1-i]                        (CHW)
// bt[ci][hk][wk][co] = w[co][Hk-1-hk][Wk-1-wk][ci]        (HWC)
template <typename T>
__global__ __launch_bounds__(256) void blocktransp_kernel(const T *__restrict__ w, T *__restrict__ bt, int Ci, int Co,
                                                          int Hk, int Wk, int hwc, int total) {
    int idx = blockIdx.x * 256 + threadIdx.x;
    if (idx >= total) return;
    const int P = Hk * Wk;
    if (!hwc) {
        int i = idx % P, co = (idx / P) % Co, ci = idx / (P * Co);
        bt[idx] = w[((size_t)co * Ci + ci) * P + (P - 1 - i)];
    } else {
        int co = idx % Co, wk = (idx / Co) % Wk, hk = (idx / (Co * Wk)) % Hk, ci = idx / (Co * P);
        bt[idx] = w[(((size_t)co * Hk + (Hk - 1 - hk)) * Wk + (Wk - 1 - wk)) * Ci + ci];
    }
}

// Channel-major weights through an LDS tile of TD output x TD input channels x P taps: a workgroup reads, for each
// of its TD output channels, the contiguous run of TD x P elements, and writes, for each of its TD input channels,
// the contiguous run of TD x P elements of the result - both sides of the transposition move whole lines, 16 bytes
// per thread where VECS says the runs are made of whole aligned chunks.  A thread keeps one chunk position of the
// run and walks down the rows, so where its elements sit in the tile (a division and a flip per element) is
// worked out once, before the loop.
template <typename T, bool VECS, int TD, int NT>
__global__ __launch_bounds__(NT) void blocktransp_tile_kernel(const T *__restrict__ w, T *__restrict__ bt, int Ci,
                                                              int Co, int P, unsigned m_p, int pitch) {
    constexpr int VEC = 16 / (int)sizeof(T), E = VECS ? VEC : 1;
    extern __shared__ __attribute__((aligned(16))) char smem[];
    T *tile = reinterpret_cast<T *>(smem);  // [TD co][pitch]
    // Tiles in groups of 2 x 2 that one XCD takes in a row (workgroups go to the eight XCDs in turn): where a tile's
    // runs end inside a 128-byte line, the neighbour that holds the rest of the line meets it in the same L2.
    const int tiles_x = (Ci + TD - 1) / TD, tiles_y = (Co + TD - 1) / TD, groups_x = (tiles_x + 1) / 2;
    const unsigned L = blockIdx.x, slot = L >> 3, group = (L & 7) + 8 * (slot >> 2), m = slot & 3;
    const int gy = group / groups_x, gx = group - gy * groups_x;
    const int tx = 2 * gx + (m & 1), ty = 2 * gy + (m >> 1);
    if (tx >= tiles_x || ty >= tiles_y) return;
    const int ci0 = tx * TD, co0 = ty * TD;
    const int nci = min(TD, Ci - ci0), nco = min(TD, Co - co0);
    const int tid = threadIdx.x;
    {
        // (a run longer than the workgroup is walked in several sweeps of c)
        const int n = nci * P, per_row = (n + E - 1) / E, span = min(per_row, NT), rstep = NT / span;
        const int row0 = tid / span;
        const size_t row_elems = (size_t)Ci * P;
        for (int c = tid - row0 * span; c < per_row && row0 < rstep; c += span) {
            const T *src = w + ((size_t)co0 * Ci + ci0) * P + row0 * row_elems + c * E;
            T *dst = tile + row0 * pitch + c * E;
            if (!VECS || c * E + E <= n) {
                typedef typename std::conditional<VECS, uint4, T>::type Piece;
                int row = row0;
                for (; row + 3 * rstep < nco; row += 4 * rstep) {
                    Piece v[4];
#pragma unroll
                    for (int u = 0; u < 4; ++u) v[u] = *reinterpret_cast<const Piece *>(src + u * rstep * row_elems);
#pragma unroll
                    for (int u = 0; u < 4; ++u) *reinterpret_cast<Piece *>(dst + u * rstep * pitch) = v[u];
                    src += 4 * rstep * row_elems;
                    dst += 4 * rstep * pitch;
                }
                for (; row < nco; row += rstep) {
                    *reinterpret_cast<Piece *>(dst) = *reinterpret_cast<const Piece *>(src);
                    src += rstep * row_elems;
                    dst += rstep * pitch;
                }
            } else {
                for (int row = row0; row < nco; row += rstep) {
                    for (int e = 0; c * E + e < n; ++e) dst[e] = src[e];
                    src += rstep * row_elems;
                    dst += rstep * pitch;
                }
            }
        }
    }
    __syncthreads();
    {
        const int n = nco * P, per_row = (n + E - 1) / E, span = min(per_row, NT), rstep = NT / span;
        const int row0 = tid / span;
        for (int c = tid - row0 * span; c < per_row && row0 < rstep; c += span) {
            int off[E];  // where the chunk's elements sit in row 0 of the tile's view for input channel 0
            unsigned co = div_magic((unsigned)(c * E), m_p), i = (unsigned)(c * E) - co * P;
#pragma unroll
            for (int e = 0; e < E; ++e) {
                off[e] = min((int)co, nco - 1) * pitch + (P - 1 - (int)i);
                if (++i == (unsigned)P) {
                    i = 0;
                    ++co;
                }
            }
            T *dst = bt + ((size_t)ci0 * Co + co0) * P + (size_t)row0 * Co * P + c * E;
            const T *t = tile + row0 * P;
            typedef typename std::conditional<VECS, uint4, T>::type Piece;
            union Chunk {
                Piece u;
                T e[E];
            };
            if (c * E + E <= n) {
                for (int row = row0; row < nci; row += rstep) {
                    Chunk v;
#pragma unroll
                    for (int e = 0; e < E; ++e) v.e[e] = t[off[e]];
                    *reinterpret_cast<Piece *>(dst) = v.u;
                    dst += (size_t)rstep * Co * P;
                    t += rstep * P;
                }
            } else {  // the run's last, partial chunk (constant indices only: others would send the chunk through memory)
                for (int row = row0; row < nci; row += rstep) {
#pragma unroll
                    for (int e = 0; e < E; ++e)
                        if (c * E + e < n) dst[e] = t[off[e]];
                    dst += (size_t)rstep * Co * P;
                    t += rstep * P;
                }
            }
        }
    }
}

template <typename T>
static int transpose2d_strided(const T *in, T *out, int N, int M, long long in_rs, long long out_rs, int batch,
                               long long in_bs, long long out_bs, long long in_base, long long out_base);

template <typename T, typename Args>
static int blocktransp(const Args *a, const char *fn) {
    if (!a || !a->weights || !a->bt_weights) {
        set_error("%s: null argument", fn);
        return 1;
    }
    int hwc = (uint8_t)a->HWC;
    if (hwc != 0 && hwc != 1) {
        printf("[%s.c] Invalid data layout (not 0 or 1)!!\n", fn);
        set_error("%s: HWC must be 0 or 1", fn);
        return 1;
    }
    if (a->Cin <= 0 || a->Cout <= 0 || a->Hk <= 0 || a->Wk <= 0) {
        set_error("%s: invalid geometry", fn);
        return 1;
    }
    if (!ensure_init()) return 2;
    size_t n = (size_t)a->Cin * a->Cout * a->Hk * a->Wk;
    Stager sg;
    const T *w = sg.in(reinterpret_cast<const T *>(a->weights), n);
    T *bt = sg.out(reinterpret_cast<T *>(a->bt_weights), n);
    if (sg.failed()) return 2;
    const int P = a->Hk * a->Wk;
    int rc = 0;
    if (hwc) {
        // per tap a strided transposition: in(co, ci) = w[co][P-1-p][ci], out(ci, co) = bt[ci][p][co]
        rc = transpose2d_strided<T>(w, bt, a->Cout, a->Cin, (long long)P * a->Cin, (long long)P * a->Cout, P,
                                    -(long long)a->Cin, (long long)a->Cout, (long long)(P - 1) * a->Cin, 0);
    } else if ((size_t)32 * (32 * P + 16 / sizeof(T)) * sizeof(T) <= 64 * 1024 && n >= 4096) {
        constexpr int VEC = 16 / (int)sizeof(T);
        const unsigned m_p = (unsigned)((((unsigned long long)1 << 32) + P - 1) / P);
        // runs of whole 16-byte chunks: every run starts on a chunk (rows of Ci x P and Co x P elements, tiles of 32 x P)
        const bool vecs = ((size_t)a->Cin * P * sizeof(T)) % 16 == 0 && ((size_t)a->Cout * P * sizeof(T)) % 16 == 0 &&
                          reinterpret_cast<uintptr_t>(w) % 16 == 0 && reinterpret_cast<uintptr_t>(bt) % 16 == 0;
        auto tile_grid = [&](int td) {  // (groups of four tiles, rounded up to eight groups)
            const long long groups = (long long)(((a->Cin + td - 1) / td + 1) / 2) * (((a->Cout + td - 1) / td + 1) / 2);
            return (unsigned)(32 * ((groups + 7) / 8));
        };
        const int pitch = 32 * P + VEC;  // rows of the tile start on 16-byte boundaries
        const size_t lds = (size_t)32 * pitch * sizeof(T);
        const dim3 grid(tile_grid(32));
        if (vecs)
            hipLaunchKernelGGL((blocktransp_tile_kernel<T, true, 32, 256>), grid, dim3(256), lds, state().stream, w, bt,
                               a->Cin, a->Cout, P, m_p, pitch);
        else
            hipLaunchKernelGGL((blocktransp_tile_kernel<T, false, 32, 256>), grid, dim3(256), lds, state().stream, w,
                               bt, a->Cin, a->Cout, P, m_p, pitch);
        rc = hip_ok(hipGetLastError(), "blocktranspose launch") ? 0 : 2;
    } else {
        if (n >= ((size_t)1 << 31)) {
            set_error("%s: tensor of 2^31 elements or more", fn);
            return sg.finish(1);
        }
        hipLaunchKernelGGL((blocktransp_kernel<T>), dim3(nblocks(n)), dim3(256), 0, state().stream, w, bt, a->Cin,
                           a->Cout, a->Hk, a->Wk, hwc, (int)n);
        rc = hip_ok(hipGetLastError(), "blocktranspose launch") ? 0 : 2;
    }
    return sg.finish(rc);
}

// ---- Transposition ------------------------------------------------------------------------

// out[j*N + i] = in[i*M + j]; 64x64 tiles through LDS so both sides coalesce.
// General form (blockIdx.z = batch b): in(i, j) = in[in_base + b*in_bs + i*in_rs + j],
// out(j, i) = out[out_base + b*out_bs + j*out_rs + i].
struct Transp2D {
    int N, M;
    long long in_rs, out_rs, in_bs, out_bs, in_base, out_base;
};

template <typename T>
__global__ __launch_bounds__(256) void transpose2d_kernel(const T *__restrict__ in, T *__restrict__ out, Transp2D g) {
    __shared__ T tile[64][65];
    in += g.in_base + (long long)blockIdx.z * g.in_bs;
    out += g.out_base + (long long)blockIdx.z * g.out_bs;
    int j0 = blockIdx.x * 64, i0 = blockIdx.y * 64;
    int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
    for (int r = ty; r < 64; r += 4) {
        int i = i0 + r, j = j0 + tx;
        if (i < g.N && j < g.M) tile[r][tx] = in[(long long)i * g.in_rs + j];
    }
    __syncthreads();
    for (int r = ty; r < 64; r += 4) {
        int j = j0 + r, i = i0 + tx;
        if (i < g.N && j < g.M) out[(long long)j * g.out_rs + i] = tile[tx][r];
    }
}

// The same with 16-byte global accesses on both sides (rows, row strides, bases and pointers multiples of 16
// bytes).  The tile is kept as dwords with a pitch of 33 (fp16: two columns per dword) or 65 (fp32), so the
// column walk of the second phase is conflict free; a thread gathers the VEC elements of its output chunk from
// VEC tile rows and stores them at once.
template <typename T>
__global__ __launch_bounds__(256) void transpose2d_vec_kernel(const T *__restrict__ in, T *__restrict__ out, Transp2D g) {
    constexpr int VEC = 16 / (int)sizeof(T), CH = 64 / VEC;  // chunks per tile row
    constexpr int PITCH = sizeof(T) == 2 ? 66 : 65;          // elements
    __shared__ __attribute__((aligned(16))) T tile[64 * PITCH];
    in += g.in_base + (long long)blockIdx.z * g.in_bs;
    out += g.out_base + (long long)blockIdx.z * g.out_bs;
    const int j0 = blockIdx.x * 64, i0 = blockIdx.y * 64;
#pragma unroll
    for (int it = 0; it < 64 * CH / 256; ++it) {
        const int item = it * 256 + threadIdx.x, r = item / CH, c = item % CH;
        const int i = i0 + r, j = j0 + c * VEC;
        if (i < g.N && j < g.M) {  // (M is a multiple of VEC: a chunk is inside or outside)
            union {
                uint4 u;
                T e[VEC];
                unsigned d[4];
            } v;
            v.u = *reinterpret_cast<const uint4 *>(in + (long long)i * g.in_rs + j);
            if (sizeof(T) == 2) {
                unsigned *row = reinterpret_cast<unsigned *>(tile + r * PITCH + c * VEC);  // 4-byte aligned
#pragma unroll
                for (int k = 0; k < 4; ++k) row[k] = v.d[k];
            } else {
#pragma unroll
                for (int k = 0; k < VEC; ++k) tile[r * PITCH + c * VEC + k] = v.e[k];
            }
        }
    }
    __syncthreads();
#pragma unroll
    for (int it = 0; it < 64 * CH / 256; ++it) {
        const int item = it * 256 + threadIdx.x, r = item / CH, c = item % CH;  // output row j0 + r, rows i0 + c*VEC ..
        const int j = j0 + r, i = i0 + c * VEC;
        if (j < g.M && i < g.N) {
            union {
                uint4 u;
                T e[VEC];
            } v;
#pragma unroll
            for (int k = 0; k < VEC; ++k) v.e[k] = tile[(c * VEC + k) * PITCH + r];
            *reinterpret_cast<uint4 *>(out + (long long)j * g.out_rs + i) = v.u;
        }
    }
}

template <typename T>
static int transpose2d_strided(const T *in, T *out, int N, int M, long long in_rs, long long out_rs, int batch,
                               long long in_bs, long long out_bs, long long in_base, long long out_base) {
    constexpr int VEC = 16 / (int)sizeof(T);
    Transp2D g = {N, M, in_rs, out_rs, in_bs, out_bs, in_base, out_base};
    dim3 grid((M + 63) / 64, (N + 63) / 64, batch);
    auto mult = [](long long v) { return v % VEC == 0; };
    const bool vec = mult(N) && mult(M) && mult(in_rs) && mult(out_rs) && mult(in_bs) && mult(out_bs) && mult(in_base) &&
                     mult(out_base) && reinterpret_cast<uintptr_t>(in) % 16 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0;
    if (vec)
        hipLaunchKernelGGL((transpose2d_vec_kernel<T>), grid, dim3(256), 0, state().stream, in, out, g);
    else
        hipLaunchKernelGGL((transpose2d_kernel<T>), grid, dim3(256), 0, state().stream, in, out, g);
    return hip_ok(hipGetLastError(), "transpose launch") ? 0 : 2;
}

template <typename T>
static int transpose2d_dev(const T *in, T *out, int N, int M) {
    return transpose2d_strided<T>(in, out, N, M, M, N, 1, 0, 0, 0, 0);
}

constexpr int MAX_ND = 8;
struct NdPerm {
    int nd;
    int out_dim[MAX_ND];    // extent of output axis i
    int in_stride[MAX_ND];  // input stride of the axis that becomes output axis i
};

// numpy.transpose semantics: output axis i is input axis axes[i].
template <typename T>
__global__ __launch_bounds__(256) void transpose_nd_kernel(const T *__restrict__ in, T *__restrict__ out, NdPerm p,
                                                           size_t total) {
    size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= total) return;
    size_t t = idx, src = 0;
    for (int i = p.nd - 1; i >= 0; --i) {
        src += (t % p.out_dim[i]) * (size_t)p.in_stride[i];
        t /= p.out_dim[i];
    }
    out[idx] = in[src];
}

template <typename T, typename Args>
static int transpose_nd(const Args *a, const char *fn) {
    if (!a || !a->in_matrix || !a->out_matrix || !a->dim || !a->transposed_axes) {
        set_error("%s: null argument", fn);
        return 1;
    }
    int nd = a->n_dim;
    if (nd < 1 || nd > MAX_ND) {
        printf("[%s] unsupported number of dimensions %d (1..%d)\n", fn, nd, MAX_ND);
        set_error("%s: unsupported number of dimensions", fn);
        return 1;
    }
    int stride[MAX_ND];
    bool seen[MAX_ND] = {false};
    size_t total = 1;
    for (int i = nd - 1; i >= 0; --i) {
        if (a->dim[i] <= 0) {
            set_error("%s: non-positive extent", fn);
            return 1;
        }
        stride[i] = (int)total;
        total *= (size_t)a->dim[i];
    }
    NdPerm p = {};
    p.nd = nd;
    for (int i = 0; i < nd; ++i) {
        int ax = a->transposed_axes[i];
        if (ax < 0 || ax >= nd || seen[ax]) {
            printf("[%s] transposed_axes is not a permutation\n", fn);
            set_error("%s: transposed_axes is not a permutation", fn);
            return 1;
        }
        seen[ax] = true;
        p.out_dim[i] = a->dim[ax];
        p.in_stride[i] = stride[ax];
    }
    if (!ensure_init()) return 2;
    Stager sg;
    const T *in = sg.in(reinterpret_cast<const T *>(a->in_matrix), total);
    T *out = sg.out(reinterpret_cast<T *>(a->out_matrix), total);
    if (sg.failed()) return 2;
    int rc;
    if (nd == 2 && a->transposed_axes[0] == 1) {
        rc = transpose2d_dev<T>(in, out, a->dim[0], a->dim[1]);
    } else {
        hipLaunchKernelGGL((transpose_nd_kernel<T>), dim3(nblocks(total)), dim3(256), 0, state().stream, in, out, p,
                           total);
        rc = hip_ok(hipGetLastError(), "transpose launch") ? 0 : 2;
    }
    return sg.finish(rc);
}

template <typename T, typename Args>
static int transpose_mat(const Args *a, const char *fn) {
    if (!a || !a->in_matrix || !a->out_matrix) {
        set_error("%s: null argument", fn);
        return 1;
    }
    if (a->N <= 0 || a->M <= 0) return 0;
    if (!ensure_init()) return 2;
    size_t total = (size_t)a->N * a->M;
    Stager sg;
    const T *in = sg.in(reinterpret_cast<const T *>(a->in_matrix), total);
    T *out = sg.out(reinterpret_cast<T *>(a->out_matrix), total);
    if (sg.failed()) return 2;
    return sg.finish(transpose2d_dev<T>(in, out, a->N, a->M));
}

// ---- Streaming helpers ---------------------------------------------------------------------

template <typename T>
__global__ __launch_bounds__(256) void copy_kernel(const T *__restrict__ a, T *__restrict__ b, size_t n) {
    size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) b[i] = a[i];
}

// 16 bytes per thread (both pointers 16-byte aligned); the last, partial chunk element by element.
template <typename T>
__global__ __launch_bounds__(256) void copy_vec_kernel(const T *__restrict__ a, T *__restrict__ b, size_t n) {
    constexpr int VEC = 16 / (int)sizeof(T);
    const size_t i = ((size_t)blockIdx.x * 256 + threadIdx.x) * VEC;
    if (i + VEC <= n) {
        *reinterpret_cast<uint4 *>(b + i) = *reinterpret_cast<const uint4 *>(a + i);
    } else {
        for (size_t e = i; e < n; ++e) b[e] = a[e];
    }
}

template <typename T>
static void launch_copy(const T *a, T *b, size_t n) {
    constexpr int VEC = 16 / (int)sizeof(T);
    if (reinterpret_cast<uintptr_t>(a) % 16 == 0 && reinterpret_cast<uintptr_t>(b) % 16 == 0)
        hipLaunchKernelGGL((copy_vec_kernel<T>), dim3(nblocks((n + VEC - 1) / VEC)), dim3(256), 0, state().stream, a, b, n);
    else
        hipLaunchKernelGGL((copy_kernel<T>), dim3(nblocks(n)), dim3(256), 0, state().stream, a, b, n);
}

__global__ __launch_bounds__(256) void copy16_kernel(const uint4 *__restrict__ a, uint4 *__restrict__ b, size_t n) {
    size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    size_t stride = (size_t)gridDim.x * 256;
    for (; i < n; i += stride) b[i] = a[i];
}

template <typename T>
__global__ __launch_bounds__(256) void fill_kernel(T *__restrict__ a, T v, size_t n) {
    size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) a[i] = v;
}

template <typename T>
__global__ __launch_bounds__(256) void add_kernel(const T *__restrict__ a, const T *__restrict__ b, T *__restrict__ c,
                                                  size_t n) {
    size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) c[i] = a[i] + b[i];
}

template <typename S, typename D>
__global__ __launch_bounds__(256) void cast_kernel(const S *__restrict__ a, D *__restrict__ b, size_t n) {
    size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) b[i] = (D)a[i];
}

// dest[c][ht][wt] = source[c][ht-U][wt-L] inside, 0 in the border (CHW; HWC alike).  A thread writes PER
// consecutive destination elements (one 16-byte store): first index decoded once, the rest by carrying.
// The elements of a chunk that come from the source are consecutive in the source (the end of a row is followed
// by the start of the next, the end of a channel by the start of the next): a chunk is one 16-byte load from the
// first of them (at element alignment - the memory system takes unaligned vector accesses) spread over the
// positions that are not border, also when it straddles rows.
template <typename T, int PER>
__global__ __launch_bounds__(256) void pad_kernel(const T *__restrict__ src, T *__restrict__ dst, int C, int H, int W,
                                                  int L, int U, int Ho, int Wo, int hwc, size_t total, size_t n_src) {
    const size_t idx0 = ((size_t)blockIdx.x * 256 + threadIdx.x) * PER;
    if (idx0 >= total) return;
    // (the host keeps the tensor below 2^32 elements: 32-bit index arithmetic)
    const unsigned i32 = (unsigned)idx0;
    int c, ht, wt;
    if (!hwc) {
        const unsigned r = i32 / (unsigned)Wo;
        wt = (int)(i32 - r * Wo);
        c = (int)(r / (unsigned)Ho);
        ht = (int)(r - (unsigned)c * Ho);
    } else {
        const unsigned r = i32 / (unsigned)C;
        c = (int)(i32 - r * C);
        ht = (int)(r / (unsigned)Wo);
        wt = (int)(r - (unsigned)ht * Wo);
    }
    unsigned mask = 0;
    size_t base = 0;
#pragma unroll
    for (int e = 0; e < PER; ++e) {
        const int h = ht - U, w = wt - L;
        if (idx0 + e < total && (unsigned)h < (unsigned)H && (unsigned)w < (unsigned)W) {
            if (mask == 0) base = hwc ? ((size_t)h * W + w) * C + c : ((size_t)c * H + h) * W + w;
            mask |= 1u << e;
        }
        if (!hwc) {
            if (++wt == Wo) {
                wt = 0;
                if (++ht == Ho) {
                    ht = 0;
                    ++c;
                }
            }
        } else {
            if (++c == C) {
                c = 0;
                if (++wt == Wo) {
                    wt = 0;
                    ++ht;
                }
            }
        }
    }
    union {
        uint4 u;
        T e[PER];
    } in, out;
    if (PER * sizeof(T) == 16 && mask != 0 && base + PER <= n_src) {
        typedef unsigned pad_u4 __attribute__((ext_vector_type(4), aligned(2)));
        const pad_u4 v = *reinterpret_cast<const pad_u4 *>(src + base);
        in.u = make_uint4(v.x, v.y, v.z, v.w);
    } else {
#pragma unroll
        for (int e = 0; e < PER; ++e) in.e[e] = (mask >> e) != 0 && base + e < n_src ? src[base + e] : (T)0;
    }
    if (mask == (1u << PER) - 1u) {
        out = in;
    } else {
        int r = 0;
#pragma unroll
        for (int e = 0; e < PER; ++e) {
            T v = (T)0;
            if (mask & (1u << e)) {
#pragma unroll
                for (int q = 0; q <= e; ++q)
                    if (q == r) v = in.e[q];
                ++r;
            }
            out.e[e] = v;
        }
    }
    if (PER * sizeof(T) == 16 && idx0 + PER <= total) {
        *reinterpret_cast<uint4 *>(dst + idx0) = out.u;
    } else {
#pragma unroll
        for (int e = 0; e < PER; ++e)
            if (idx0 + e < total) dst[idx0 + e] = out.e[e];
    }
}

// The same result with far fewer instructions per chunk, for rows of at least one chunk.  Both layouts are one
// case: NR = groups x Ho rows of WoE elements, of which rows U .. U+H-1 of a group hold WE source elements from
// column LE on (channel-major: groups = C, WoE = Wo; channel-last: one group, rows of Wo x C).  The source elements
// that a run of destination elements takes are consecutive, so a workgroup copies the aligned 16-byte pieces of the
// source that cover its 256 chunks into LDS (one coalesced load per thread), and a thread picks its chunk out of
// them: validity is a bit mask built from the two row segments a chunk can touch, and the e-th valid element is the
// (number of valid elements before it)-th after the chunk's first.  The row and column of a workgroup's first
// element come from one division per workgroup; a thread's own from reciprocal multiplications on the small rest.
struct PadRows {
    int Ho, H, U, WoE, WE, LE;
    unsigned m_wo, m_ho;  // ceil(2^32 / WoE), ceil(2^32 / Ho)
};

template <typename T>
__global__ __launch_bounds__(256) void pad_rows_kernel(const T *__restrict__ src, T *__restrict__ dst, PadRows g,
                                                       unsigned total, unsigned n_src) {
    constexpr int PER = 16 / (int)sizeof(T);
    __shared__ __attribute__((aligned(16))) T span[(256 + 2) * PER];
    // valid source elements before destination position (group c, row ht, column wt)
    auto before = [&](unsigned c, int ht, int wt) {
        const int rows = min(max(ht - g.U, 0), g.H);
        const int cols = (unsigned)(ht - g.U) < (unsigned)g.H ? min(max(wt - g.LE, 0), g.WE) : 0;
        return (c * g.H + rows) * (unsigned)g.WE + cols;
    };
    const unsigned B = blockIdx.x * (256u * PER);
    const unsigned r_B = B / (unsigned)g.WoE, wt_B = B - r_B * g.WoE;
    const unsigned c_B = r_B / (unsigned)g.Ho, ht_B = r_B - c_B * g.Ho;
    const unsigned s_lo = before(c_B, (int)ht_B, (int)wt_B) & ~(unsigned)(PER - 1);
    // the pieces of the source this workgroup's chunks can take from: at most 256 x PER elements and two ragged
    // ends - a piece per thread and two more, both loads on their way before either is waited for (what lies
    // beyond the source comes from a piece of zeros: a load under a condition would wait on its own)
    {
        typedef const PatchPiece __attribute__((address_space(1))) *GlobalPiece;
        const unsigned at0 = s_lo + threadIdx.x * PER, at1 = s_lo + (256 + threadIdx.x) * PER;
        const bool more = threadIdx.x < 2;
        const PatchPiece v0 = *(at0 + PER <= n_src ? (GlobalPiece)(src + at0) : (GlobalPiece)&patch_zero);
        const PatchPiece v1 = *(more && at1 + PER <= n_src ? (GlobalPiece)(src + at1) : (GlobalPiece)&patch_zero);
        *reinterpret_cast<PatchPiece *>(span + threadIdx.x * PER) = v0;
        if (more) *reinterpret_cast<PatchPiece *>(span + (256 + threadIdx.x) * PER) = v1;
        // (the tensor's last, partial piece, element by element)
        if (at0 < n_src && at0 + PER > n_src)
            for (int e = 0; at0 + e < n_src; ++e) span[threadIdx.x * PER + e] = src[at0 + e];
        if (more && at1 < n_src && at1 + PER > n_src)
            for (int e = 0; at1 + e < n_src; ++e) span[(256 + threadIdx.x) * PER + e] = src[at1 + e];
    }
    __syncthreads();
    const unsigned idx0 = B + threadIdx.x * PER;
    if (idx0 >= total) return;
    // this thread's row and column: a few rows below the workgroup's first
    const unsigned x = wt_B + threadIdx.x * PER, dr = div_magic(x, g.m_wo);
    const int wt = (int)(x - dr * g.WoE);
    const unsigned y = ht_B + dr, dc = div_magic(y, g.m_ho);
    const int ht = (int)(y - dc * g.Ho);
    const unsigned c = c_B + dc;
    // valid positions of the chunk: the rest of this row, then the start of the next
    const int n1 = min(PER, g.WoE - wt), ht2 = ht + 1 == g.Ho ? 0 : ht + 1;
    unsigned mask = 0;
    if ((unsigned)(ht - g.U) < (unsigned)g.H) {
        const int lo = max(g.LE - wt, 0), hi = min(g.LE + g.WE - wt, n1);
        if (hi > lo) mask = ((1u << hi) - 1u) & ~((1u << lo) - 1u);
    }
    if (n1 < PER && (unsigned)(ht2 - g.U) < (unsigned)g.H) {
        const int lo = n1 + g.LE, hi = min(n1 + g.LE + g.WE, PER);
        if (hi > lo) mask |= ((1u << hi) - 1u) & ~((1u << lo) - 1u);
    }
    const T *from = span + (before(c, ht, wt) - s_lo);
    union {
        uint4 u;
        T e[PER];
    } out;
#pragma unroll
    for (int e = 0; e < PER; ++e) {
        const T v = from[__popc(mask & ((1u << e) - 1u))];
        out.e[e] = (mask >> e) & 1u ? v : (T)0;
    }
    if (idx0 + PER <= total) {
        *reinterpret_cast<uint4 *>(dst + idx0) = out.u;
    } else {
#pragma unroll
        for (int e = 0; e < PER; ++e)
            if (idx0 + e < total) dst[idx0 + e] = out.e[e];
    }
}

template <typename T, typename Args>
static int pad_step(const Args *a, const char *fn) {
    if (!a || !a->source || !a->dest) {
        set_error("%s: null argument", fn);
        return 1;
    }
    if (a->HWC_lay != 0 && a->HWC_lay != 1) {
        printf("[%s] HWC layout not implemented!!", fn);
        set_error("%s: HWC_lay must be 0 or 1", fn);
        return 1;
    }
    if (a->C <= 0 || a->H <= 0 || a->W <= 0 || a->T_LPAD < 0 || a->T_RPAD < 0 || a->T_UPAD < 0 || a->T_DPAD < 0) {
        set_error("%s: invalid geometry", fn);
        return 1;
    }
    if (!ensure_init()) return 2;
    int Ho = a->H + a->T_UPAD + a->T_DPAD, Wo = a->W + a->T_LPAD + a->T_RPAD;
    size_t total = (size_t)a->C * Ho * Wo;
    if (total >= ((size_t)1 << 32)) {
        set_error("%s: tensor of 2^32 elements or more", fn);
        return 1;
    }
    Stager sg;
    const T *s = sg.in(reinterpret_cast<const T *>(a->source), (size_t)a->C * a->H * a->W);
    T *d = sg.out(reinterpret_cast<T *>(a->dest), total);
    if (sg.failed()) return 2;
    constexpr int VEC = 16 / (int)sizeof(T);
    const size_t n_src = (size_t)a->C * a->H * a->W;
    // rows of at least a chunk, short enough for the reciprocal divisions (exact below 2^16) of a row or column
    // index a workgroup's 256 chunks further on
    const long long WoE = a->HWC_lay ? (long long)Wo * a->C : Wo;
    const bool rows_form = reinterpret_cast<uintptr_t>(d) % 16 == 0 && reinterpret_cast<uintptr_t>(s) % 16 == 0 &&
                           WoE >= VEC && WoE + 256 * VEC < 65536 && Ho + 256 * VEC < 65536 && state().gemm_path != 1;
    if (rows_form) {
        PadRows g;
        g.Ho = Ho; g.H = a->H; g.U = a->T_UPAD;
        g.WoE = (int)WoE; g.WE = a->HWC_lay ? a->W * a->C : a->W; g.LE = a->HWC_lay ? a->T_LPAD * a->C : a->T_LPAD;
        g.m_wo = (unsigned)((((unsigned long long)1 << 32) + g.WoE - 1) / g.WoE);
        g.m_ho = (unsigned)((((unsigned long long)1 << 32) + Ho - 1) / Ho);
        hipLaunchKernelGGL((pad_rows_kernel<T>), dim3(nblocks((total + VEC - 1) / VEC)), dim3(256), 0, state().stream, s, d,
                           g, (unsigned)total, (unsigned)n_src);
    } else if (reinterpret_cast<uintptr_t>(d) % 16 == 0)
        hipLaunchKernelGGL((pad_kernel<T, VEC>), dim3(nblocks((total + VEC - 1) / VEC)), dim3(256), 0, state().stream, s, d,
                           a->C, a->H, a->W, a->T_LPAD, a->T_UPAD, Ho, Wo, a->HWC_lay, total, n_src);
    else
        hipLaunchKernelGGL((pad_kernel<T, 1>), dim3(nblocks(total)), dim3(256), 0, state().stream, s, d, a->C, a->H, a->W,
                           a->T_LPAD, a->T_UPAD, Ho, Wo, a->HWC_lay, total, n_src);
    return sg.finish(hip_ok(hipGetLastError(), "pad launch") ? 0 : 2);
}

// Layout change of one tensor: transpose [rows x cols] into the caller's buffer,
// then copy the buffer back over the tensor, as the reference does
// (lib/sources/pulp_train_utils_fp32.c:821-927).
template <typename T>
static int relayout_one(T *tensor, T *buffer, int rows, int cols, Stager &sg) {
    size_t n = (size_t)rows * cols;
    T *t = sg.inout(tensor, n);
    T *b = sg.out(buffer, n);
    if (sg.failed()) return 2;
    int rc = transpose2d_dev<T>(t, b, rows, cols);
    if (rc) return rc;
    launch_copy<T>(b, t, n);
    return hip_ok(hipGetLastError(), "copy launch") ? 0 : 2;
}

template <typename T, typename Args>
static int relayout(const Args *a, bool to_hwc, const char *fn) {
    if (!a || !a->tensor || !a->transp_buffer) {
        set_error("%s: null argument", fn);
        return 1;
    }
    // the reference narrows C/H/W to 16 bits (lib/sources/pulp_train_utils_fp32.c:825-827)
    int C = (uint16_t)a->tensor->C, H = (uint16_t)a->tensor->H, W = (uint16_t)a->tensor->W;
    if (C == 0 || H == 0 || W == 0) return 0;
    if (!ensure_init()) return 2;
    int rows = to_hwc ? C : H * W, cols = to_hwc ? H * W : C;
    Stager sg;
    int rc = 0;
    if ((uint8_t)a->transpose_data == 1) {
        if (!a->tensor->data) {
            set_error("%s: transpose_data=1 with null data", fn);
            return 1;
        }
        rc = relayout_one<T>(reinterpret_cast<T *>(a->tensor->data), reinterpret_cast<T *>(a->transp_buffer), rows,
                             cols, sg);
    }
    if (rc == 0 && (uint8_t)a->transpose_grad == 1) {
        if (!a->tensor->diff) {
            set_error("%s: transpose_grad=1 with null diff", fn);
            return 1;
        }
        rc = relayout_one<T>(reinterpret_cast<T *>(a->tensor->diff), reinterpret_cast<T *>(a->transp_buffer), rows,
                             cols, sg);
    }
    return sg.finish(rc);
}

template <typename T>
static int copy_step(const T *from, T *to, int size) {
    if (size <= 0) return 0;
    if (!from || !to) {
        set_error("copy: null argument");
        return 1;
    }
    if (!ensure_init()) return 2;
    Stager sg;
    const T *a = sg.in(from, (size_t)size);
    T *b = sg.out(to, (size_t)size);
    if (sg.failed()) return 2;
    launch_copy<T>(a, b, (size_t)size);
    return sg.finish(hip_ok(hipGetLastError(), "copy launch") ? 0 : 2);
}

template <typename T>
static int fill_step(T *to, T value, int size) {
    if (size <= 0) return 0;
    if (!to) {
        set_error("set_to_value: null argument");
        return 1;
    }
    if (!ensure_init()) return 2;
    Stager sg;
    T *b = sg.out(to, (size_t)size);
    if (sg.failed()) return 2;
    hipLaunchKernelGGL((fill_kernel<T>), dim3(nblocks(size)), dim3(256), 0, state().stream, b, value, (size_t)size);
    return sg.finish(hip_ok(hipGetLastError(), "fill launch") ? 0 : 2);
}

template <typename T>
static int add_step(const T *x, const T *y, T *z, int size) {
    if (size <= 0) return 0;
    if (!x || !y || !z) {
        set_error("vect_sum: null argument");
        return 1;
    }
    if (!ensure_init()) return 2;
    Stager sg;
    const T *a = sg.in(x, (size_t)size);
    const T *b = sg.in(y, (size_t)size);
    T *c = sg.out(z, (size_t)size);
    if (sg.failed()) return 2;
    hipLaunchKernelGGL((add_kernel<T>), dim3(nblocks(size)), dim3(256), 0, state().stream, a, b, c, (size_t)size);
    return sg.finish(hip_ok(hipGetLastError(), "add launch") ? 0 : 2);
}

template <typename S, typename D>
static int cast_step(const S *x, D *y, int size) {
    if (size <= 0) return 0;
    if (!x || !y) {
        set_error("cast: null argument");
        return 1;
    }
    if (!ensure_init()) return 2;
    Stager sg;
    const S *a = sg.in(x, (size_t)size);
    D *b = sg.out(y, (size_t)size);
    if (sg.failed()) return 2;
    hipLaunchKernelGGL((cast_kernel<S, D>), dim3(nblocks(size)), dim3(256), 0, state().stream, a, b, (size_t)size);
    return sg.finish(hip_ok(hipGetLastError(), "cast launch") ? 0 : 2);
}

}  // namespace ptl

// ---- C ABI ---------------------------------------------------------------------------------
using ptl::half_t;
using ptl::set_status;

extern "C" {

int ptl_conv_dw_fp32_fw_batched(const struct DepthWise_Conv_args *a, int ns) {
    return ptl::dw_step<float>(a, ns, STEP_FW, a ? a->stride_h : 1, a ? a->stride_w : 1, "pulp_conv_dw_fp32_fw_cl");
}
int ptl_conv_dw_fp32_wg_batched(const struct DepthWise_Conv_args *a, int ns) {
    return ptl::dw_step<float>(a, ns, STEP_WGT_GRAD, a ? a->stride_h : 1, a ? a->stride_w : 1,
                               "pulp_conv_dw_fp32_bw_param_grads_cl");
}
int ptl_conv_dw_fp32_ig_batched(const struct DepthWise_Conv_args *a, int ns) {
    return ptl::dw_step<float>(a, ns, STEP_IN_GRAD, a ? a->stride_h : 1, a ? a->stride_w : 1,
                               "pulp_conv_dw_fp32_bw_input_grads_cl");
}
int ptl_conv_dw_fp16_fw_batched(const struct DepthWise_Conv_args_fp16 *a, int ns) {
    return ptl::dw_step<half_t>(a, ns, STEP_FW, 1, 1, "pulp_conv_dw_fp16_fw_cl");
}
int ptl_conv_dw_fp16_wg_batched(const struct DepthWise_Conv_args_fp16 *a, int ns) {
    return ptl::dw_step<half_t>(a, ns, STEP_WGT_GRAD, 1, 1, "pulp_conv_dw_fp16_bw_param_grads_cl");
}

// Allocation-free twin of ptl_conv_dw_fp16_wg_batched: same kernels, partial sums in the fixed device array.
int ptl_conv_dw_fp16_wg_noalloc(const struct DepthWise_Conv_args_fp16 *a, int ns) {
    ptl::State &st = ptl::state();
    if (!st.ready) {
        ptl::set_error("ptl_conv_dw_fp16_wg_noalloc: call ptl_init() first (initialisation may allocate, this call may not)");
        return 1;
    }
    float *buf = st.device >= 0 && st.device < ptl::DW_NOALLOC_MAX_DEVICES ? ptl::g_dw_wg_scratch_ptr[st.device] : nullptr;
    if (!buf) {
        ptl::set_error("ptl_conv_dw_fp16_wg_noalloc: no fixed buffer on device %d", st.device);
        return 2;
    }
    return ptl::dw_step<half_t>(a, ns, STEP_WGT_GRAD, 1, 1, "ptl_conv_dw_fp16_wg_noalloc", buf, ptl::DW_NOALLOC_BYTES);
}
int ptl_conv_dw_fp16_ig_batched(const struct DepthWise_Conv_args_fp16 *a, int ns) {
    return ptl::dw_step<half_t>(a, ns, STEP_IN_GRAD, 1, 1, "pulp_conv_dw_fp16_bw_input_grads_cl");
}

void pulp_im2row_fp32(void *p) {
    set_status(ptl::patch_build<float>(static_cast<const struct im2col_args *>(p), 0, "pulp_im2col_fp32"));
}
void pulp_im2col_fp32(void *p) {
    set_status(ptl::patch_build<float>(static_cast<const struct im2col_args *>(p), 1, "pulp_im2col_fp32"));
}
void pulp_im2row_fp16(void *p) {
    set_status(ptl::patch_build<half_t>(static_cast<const struct im2col_args_fp16 *>(p), 0, "pulp_im2col_fp16"));
}
void pulp_im2col_fp16(void *p) {
    set_status(ptl::patch_build<half_t>(static_cast<const struct im2col_args_fp16 *>(p), 1, "pulp_im2col_fp16"));
}
void pulp_blocktransp_fp32(void *p) {
    set_status(ptl::blocktransp<float>(static_cast<const struct blocktransp_args *>(p), "pulp_blocktransp_fp32"));
}
void pulp_blocktransp_fp16(void *p) {
    set_status(
        ptl::blocktransp<half_t>(static_cast<const struct blocktransp_args_fp16 *>(p), "pulp_blocktransp_fp16"));
}

void transpose_matrix(void *p) {
    set_status(ptl::transpose_mat<float>(static_cast<const struct transp_args *>(p), "transpose_matrix"));
}
void transpose_matrix_fp16(void *p) {
    set_status(ptl::transpose_mat<half_t>(static_cast<const struct transp_args_fp16 *>(p), "transpose_matrix_fp16"));
}
void transpose(void *p) {
    set_status(ptl::transpose_nd<float>(static_cast<const struct transp_args *>(p), "transpose"));
}
void transpose_fp16(void *p) {
    set_status(ptl::transpose_nd<half_t>(static_cast<const struct transp_args_fp16 *>(p), "transpose_fp16"));
}

void copy(void *p) {
    const struct copy_args *a = static_cast<const struct copy_args *>(p);
    set_status(a ? ptl::copy_step<float>(a->from, a->to, a->size) : 1);
}
void copy_fp16(void *p) {
    const struct copy_args_fp16 *a = static_cast<const struct copy_args_fp16 *>(p);
    set_status(a ? ptl::copy_step<half_t>(reinterpret_cast<const half_t *>(a->from),
                                          reinterpret_cast<half_t *>(a->to), a->size)
                 : 1);
}
void set_to_value(void *p) {
    const struct set_to_value_args *a = static_cast<const struct set_to_value_args *>(p);
    set_status(a ? ptl::fill_step<float>(a->to, a->value, a->size) : 1);
}
void set_to_value_fp16(void *p) {
    const struct set_to_value_args_fp16 *a = static_cast<const struct set_to_value_args_fp16 *>(p);
    set_status(a ? ptl::fill_step<half_t>(reinterpret_cast<half_t *>(a->to), (half_t)a->value, a->size) : 1);
}
void vect_sum(void *p) {
    const struct vect_sum_args *a = static_cast<const struct vect_sum_args *>(p);
    set_status(a ? ptl::add_step<float>(a->op_1, a->op_2, a->dest, a->size) : 1);
}
void vect_sum_fp16(void *p) {
    const struct vect_sum_args_fp16 *a = static_cast<const struct vect_sum_args_fp16 *>(p);
    set_status(a ? ptl::add_step<half_t>(reinterpret_cast<const half_t *>(a->op_1),
                                         reinterpret_cast<const half_t *>(a->op_2),
                                         reinterpret_cast<half_t *>(a->dest), a->size)
                 : 1);
}
void cast_fp16_tensor_to_fp32(void *p) {
    const struct cast_16t32_args *a = static_cast<const struct cast_16t32_args *>(p);
    set_status(a ? ptl::cast_step<half_t, float>(reinterpret_cast<const half_t *>(a->source), a->destination, a->size)
                 : 1);
}
void cast_fp32_tensor_to_fp16(void *p) {
    const struct cast_32t16_args *a = static_cast<const struct cast_32t16_args *>(p);
    set_status(a ? ptl::cast_step<float, half_t>(a->source, reinterpret_cast<half_t *>(a->destination), a->size) : 1);
}
void HWC_to_CHW(void *p) {
    set_status(ptl::relayout<float>(static_cast<const struct layout_args *>(p), false, "HWC_to_CHW"));
}
void CHW_to_HWC(void *p) {
    set_status(ptl::relayout<float>(static_cast<const struct layout_args *>(p), true, "CHW_to_HWC"));
}
void HWC_to_CHW_fp16(void *p) {
    set_status(ptl::relayout<half_t>(static_cast<const struct layout_args_fp16 *>(p), false, "HWC_to_CHW_fp16"));
}
void CHW_to_HWC_fp16(void *p) {
    set_status(ptl::relayout<half_t>(static_cast<const struct layout_args_fp16 *>(p), true, "CHW_to_HWC_fp16"));
}
void pad_tensor(void *p) {
    set_status(ptl::pad_step<float>(static_cast<const struct pad_args *>(p), "pad_tensor"));
}
void pad_tensor_fp16(void *p) {
    set_status(ptl::pad_step<half_t>(static_cast<const struct pad_args_fp16 *>(p), "pad_tensor_fp16"));
}

int ptl_copy_bytes(const void *src, void *dst, long bytes) {
    if (!src || !dst || bytes < 0 || bytes % 16 != 0) {
        ptl::set_error("ptl_copy_bytes: size must be a non-negative multiple of 16");
        return 1;
    }
    if (bytes == 0) return 0;
    if (!ptl::ensure_init()) return 2;
    size_t n = (size_t)bytes / 16;
    unsigned blocks = (unsigned)((n + 255) / 256);
    unsigned cap = (unsigned)ptl::state().num_cu * 16;
    if (blocks > cap) blocks = cap;
    hipLaunchKernelGGL(ptl::copy16_kernel, dim3(blocks), dim3(256), 0, ptl::state().stream,
                       static_cast<const uint4 *>(src), static_cast<uint4 *>(dst), n);
    return ptl::hip_ok(hipGetLastError(), "copy launch") ? 0 : 2;
}

}  // extern "C"
