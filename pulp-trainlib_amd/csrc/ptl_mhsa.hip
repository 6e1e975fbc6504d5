// Multi-head self-attention training step, fp32 (lib/sources/pulp_mhsa_fp32.c:20 forward, :648 backward)
// and the row softmax it is built on (lib/sources/pulp_act_fp32.c:187, :335).
//
// Tensors (L = sequence length, E = token size, F = heads x head size H; tokens are COLUMNS):
//   input/output E x L, q/k/v/attention_map F x L, softmax_buffer heads x L x L (row = query, column = key),
//   coeff_in_* stored E x F with gradients F x E, coeff_out E x F.
// The reference writes a transposed copy of an operand into a scratch buffer before most products; here the
// projections run on the index-map GEMM (which reads operands in place in either orientation) and the
// per-head part runs in three fused kernels that keep a 32-query (or 32-key) tile of the L x L score matrix
// in LDS:
//   forward      scores -> approximate-exponential softmax -> probabilities (saved) -> value mix
//   backward I   per query tile: dP = dA^T v, softmax backward, dq
//   backward II  per key tile:   dv = dA P, dk = q dS
// MFMA: v_mfma_f32_32x32x2_f32.  Rows of the F x L tensors are L floats long (197 in ViT-Tiny), so nothing
// here assumes 16-byte alignment of a row: global accesses are 4-byte, consecutive lanes on consecutive
// addresses.
#include <float.h>

#include "ptl_api.h"
#include "ptl_host.hpp"
#include "ptl_internal.h"
#include "ptl_structs.h"

namespace ptl {

typedef float mh_f32x16 __attribute__((ext_vector_type(16)));

constexpr int ATT_NT = 256;  // threads of an attention workgroup (4 waves)
constexpr int ATT_CK = 64;   // contraction columns staged per chunk
constexpr int ATT_VP = ATT_CK + 1;
constexpr int ATT_RP = 33;   // pitch of a parked 32 x 32 accumulator tile

// exp(x) by writing a scaled, shifted x into the exponent field (fastexp_gist,
// lib/sources/pulp_train_utils_fp32.c:1223, constants lib/include/pulp_train_defines.h:85-88).
// Multiply and add are rounded separately, as in the reference's golden model.
__device__ inline float fastexp_gist(float x) {
    x = __fadd_rn(__fmul_rn(12102203.17133801f, x), 1064986823.010288f);
    if (x < 8388608.f || x > 2139095040.f) x = (x < 8388608.f) ? 0.0f : 2139095040.f;
    return __builtin_bit_cast(float, (uint32_t)x);
}

// 1/sqrt by the magic-constant estimate and one Newton step (q_rsqrt,
// lib/sources/pulp_train_utils_fp32.c:1234; 32-bit integer as on the reference's target).
static float q_rsqrt_host(float number) {
    float x2 = number * 0.5f, y = number;
    int32_t i = __builtin_bit_cast(int32_t, y);
    i = 0x5f3759df - (i >> 1);
    y = __builtin_bit_cast(float, i);
    return y * (1.5f - (x2 * y * y));
}

__device__ inline float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o));
    return v;
}
__device__ inline float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
    return v;
}

// S[r][c] = scale * sum_d R[d][r0 + r] * Cm[d][c] for 32 rows r and every column c < L, into the LDS tile
// S[32][LP].  R and Cm are [H][L] in global memory (consecutive lanes read consecutive r or c).  Each wave owns
// every fourth 32-column block; the 32 row fragments stay in registers for all of them.
template <int HMAX>
__device__ inline void scores_to_lds(const float *__restrict__ R, const float *__restrict__ Cm, int L, int H,
                                     int r0, float scale, float *S, int LP) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int l32 = lane & 31, half = lane >> 5;
    constexpr int STEPS = HMAX / 2;
    float af[STEPS];
    const int r = r0 + l32;
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
        const int d = 2 * s + half;
        af[s] = (r < L && d < H) ? R[(size_t)d * L + r] : 0.f;
    }
    const int CB = (L + 31) / 32;
    for (int cb = wave; cb < CB; cb += 4) {
        const int c = cb * 32 + l32;
        float bf[STEPS];
#pragma unroll
        for (int s = 0; s < STEPS; ++s) {
            const int d = 2 * s + half;
            bf[s] = (c < L && d < H) ? Cm[(size_t)d * L + c] : 0.f;
        }
        mh_f32x16 acc = {0};
#pragma unroll
        for (int s = 0; s < STEPS; ++s) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(af[s], bf[s], acc, 0, 0, 0);
#pragma unroll
        for (int v = 0; v < 16; ++v) S[(8 * (v / 4) + 4 * half + (v % 4)) * LP + c] = acc[v] * scale;
    }
}

// out[d][r0 + r] = sum_c V[d][c] * S[r][c] for d < H, with S the LDS tile (columns >= L hold zeros up to the
// chunk boundary) and V [H][L] in global memory, staged through LDS in chunks of ATT_CK columns (fetched
// row-wise, read column-wise).  The 32-row blocks of d and, when there are fewer than four of them, ranges
// of the contraction are dealt to the four waves; partial tiles meet in LDS.
template <int HMAX>
__device__ inline void mix_from_lds(const float *__restrict__ V, const float *S, int LP, int L, int H, int r0,
                                    float *__restrict__ out, float *vbuf, float *red) {
    constexpr int DB = HMAX / 32, KS = 4 / DB;
    constexpr int PER = HMAX * ATT_CK / ATT_NT;
    constexpr int SPW = (ATT_CK / 2) / KS;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l32 = lane & 31, half = lane >> 5;
    const int db = wave % DB, ks = wave / DB;
    float stage[PER];
    auto fetch = [&](int c0) {
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            const int idx = tid + ATT_NT * i, d = idx >> 6, c = c0 + (idx & 63);
            stage[i] = (d < H && c < L) ? V[(size_t)d * L + c] : 0.f;
        }
    };
    const int chunks = (L + ATT_CK - 1) / ATT_CK;
    mh_f32x16 acc = {0};
    fetch(0);
    for (int ch = 0; ch < chunks; ++ch) {
        __syncthreads();  // the previous chunk has been consumed
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            const int idx = tid + ATT_NT * i;
            vbuf[(idx >> 6) * ATT_VP + (idx & 63)] = stage[i];
        }
        __syncthreads();
        if (ch + 1 < chunks) fetch((ch + 1) * ATT_CK);
#pragma unroll
        for (int s = 0; s < SPW; ++s) {
            const int kk = 2 * (ks * SPW + s) + half;
            const float a = vbuf[(db * 32 + l32) * ATT_VP + kk];
            const float b = S[l32 * LP + ch * ATT_CK + kk];
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, acc, 0, 0, 0);
        }
    }
#pragma unroll
    for (int v = 0; v < 16; ++v) red[(wave * 32 + 8 * (v / 4) + 4 * half + (v % 4)) * ATT_RP + l32] = acc[v];
    __syncthreads();
    for (int idx = tid; idx < HMAX * 32; idx += ATT_NT) {
        const int d = idx >> 5, rr = idx & 31;
        float s = 0.f;
#pragma unroll
        for (int k2 = 0; k2 < KS; ++k2) s += red[((k2 * DB + (d >> 5)) * 32 + (d & 31)) * ATT_RP + rr];
        if (d < H && r0 + rr < L) out[(size_t)d * L + r0 + rr] = s;
    }
}

struct AttnArgs {
    const float *q, *k, *v;  // [ns][F][L]
    const float *p;          // probabilities [ns][heads][L][L]   (backward)
    const float *da;         // attention_map gradient [ns][F][L]  (backward)
    const float *dp;         // probability gradient               (backward II)
    const float *rs;         // row sums of dP.P [ns][heads][L]    (backward II)
    float *o0, *o1, *o2;     // kernel outputs (see each kernel)
    int L, H, heads, F, LP;
    float scale;
};

// Forward: o0 = probabilities, o1 = attention_map.  grid (query tiles, heads, samples).
template <int HMAX>
__global__ __launch_bounds__(ATT_NT) void attn_fw_kernel(AttnArgs a) {
    extern __shared__ float att_lds[];
    float *S = att_lds, *vbuf = S + 32 * a.LP, *red = vbuf + HMAX * ATT_VP;
    const int r0 = blockIdx.x * 32, h = blockIdx.y, b = blockIdx.z, L = a.L;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const size_t hoff = ((size_t)b * a.F + (size_t)h * a.H) * L;
    scores_to_lds<HMAX>(a.q + hoff, a.k + hoff, L, a.H, r0, a.scale, S, a.LP);
    __syncthreads();
    // softmax of each row over the keys (lib/sources/pulp_act_fp32.c:187-225): max, approximate exponential of
    // the difference, sum, division
    float *P = a.o0 + ((size_t)b * a.heads + h) * L * L;
    for (int row = wave; row < 32; row += 4) {
        float *srow = S + row * a.LP;
        float mx = -FLT_MAX;
        for (int c = lane; c < L; c += 64) mx = fmaxf(mx, srow[c]);
        mx = wave_max(mx);
        float sum = 0.f;
        for (int c = lane; c < L; c += 64) {
            const float e = fastexp_gist(srow[c] - mx);
            srow[c] = e;
            sum += e;
        }
        sum = wave_sum(sum);
        const bool live = r0 + row < L;
        for (int c = lane; c < L; c += 64) {
            const float pv = srow[c] / sum;
            srow[c] = pv;
            if (live) P[(size_t)(r0 + row) * L + c] = pv;
        }
        for (int c = L + lane; c < a.LP - 1; c += 64) srow[c] = 0.f;
    }
    __syncthreads();
    mix_from_lds<HMAX>(a.v + hoff, S, a.LP, L, a.H, r0, a.o1 + hoff, vbuf, red);
}

// Backward, query side: o0 = dP (softmax_buffer gradient), o1 = dq, o2 = row sums of dP.P.
template <int HMAX>
__global__ __launch_bounds__(ATT_NT) void attn_bw_query_kernel(AttnArgs a) {
    extern __shared__ float att_lds[];
    float *S = att_lds, *vbuf = S + 32 * a.LP, *red = vbuf + HMAX * ATT_VP;
    const int r0 = blockIdx.x * 32, h = blockIdx.y, b = blockIdx.z, L = a.L;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const size_t hoff = ((size_t)b * a.F + (size_t)h * a.H) * L;
    const size_t poff = ((size_t)b * a.heads + h) * L * L;
    // dP[query][key] = sum_d dA[d][query] v[d][key]   (lib/sources/pulp_mhsa_fp32.c:958-1060)
    scores_to_lds<HMAX>(a.da + hoff, a.v + hoff, L, a.H, r0, 1.0f, S, a.LP);
    __syncthreads();
    // softmax backward (lib/sources/pulp_act_fp32.c:335-390) and the scaling (:1176-1183)
    for (int row = wave; row < 32; row += 4) {
        float *srow = S + row * a.LP;
        const bool live = r0 + row < L;
        const float *prow = a.p + poff + (size_t)(r0 + row) * L;
        float *dprow = a.o0 + poff + (size_t)(r0 + row) * L;
        float sum = 0.f;
        if (live)
            for (int c = lane; c < L; c += 64) sum += srow[c] * prow[c];
        sum = wave_sum(sum);
        for (int c = lane; c < L; c += 64) {
            const float g = srow[c];
            float ds = 0.f;
            if (live) {
                dprow[c] = g;
                ds = ((g - sum) * prow[c]) * a.scale;
            }
            srow[c] = ds;
        }
        for (int c = L + lane; c < a.LP - 1; c += 64) srow[c] = 0.f;
        if (live && lane == 0) a.o2[((size_t)b * a.heads + h) * L + r0 + row] = sum;
    }
    __syncthreads();
    // dq[d][query] = sum_key k[d][key] dS[query][key]   (:1342-1360)
    mix_from_lds<HMAX>(a.k + hoff, S, a.LP, L, a.H, r0, a.o1 + hoff, vbuf, red);
}

// Backward, key side: o0 = dv, o1 = dk for a tile of 32 keys.
//   dv[d][key] = sum_query dA[d][query] P[query][key]                         (:884-902)
//   dk[d][key] = sum_query q[d][query] dS[query][key], dS = (dP - rs) P scale  (:1244-1330)
// dA and q are staged through LDS chunk by chunk of the queries; P and dP are read from global memory with
// the keys on consecutive lanes.
template <int HMAX>
__global__ __launch_bounds__(ATT_NT) void attn_bw_key_kernel(AttnArgs a) {
    extern __shared__ float att_lds[];
    float *abuf = att_lds, *qbuf = abuf + HMAX * ATT_VP, *red = qbuf + HMAX * ATT_VP;
    constexpr int DB = HMAX / 32, KS = 4 / DB;
    constexpr int PER = HMAX * ATT_CK / ATT_NT;
    constexpr int SPW = (ATT_CK / 2) / KS;
    const int c0 = blockIdx.x * 32, h = blockIdx.y, b = blockIdx.z, L = a.L, H = a.H;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l32 = lane & 31, half = lane >> 5;
    const int db = wave % DB, ks = wave / DB;
    const size_t hoff = ((size_t)b * a.F + (size_t)h * H) * L;
    const size_t poff = ((size_t)b * a.heads + h) * L * L;
    const float *dA = a.da + hoff, *Q = a.q + hoff, *P = a.p + poff, *dP = a.dp + poff;
    const float *rs = a.rs + ((size_t)b * a.heads + h) * L;
    const int c = c0 + l32;

    float sa[PER], sq[PER], pf[SPW], sf[SPW];
    auto fetch = [&](int q0) {
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            const int idx = tid + ATT_NT * i, d = idx >> 6, r = q0 + (idx & 63);
            const bool ok = d < H && r < L;
            sa[i] = ok ? dA[(size_t)d * L + r] : 0.f;
            sq[i] = ok ? Q[(size_t)d * L + r] : 0.f;
        }
#pragma unroll
        for (int s = 0; s < SPW; ++s) {
            const int r = q0 + 2 * (ks * SPW + s) + half;
            const bool ok = r < L && c < L;
            const float pv = ok ? P[(size_t)r * L + c] : 0.f;
            const float g = ok ? dP[(size_t)r * L + c] : 0.f;
            const float rr = ok ? rs[r] : 0.f;
            pf[s] = pv;
            sf[s] = ((g - rr) * pv) * a.scale;
        }
    };
    const int chunks = (L + ATT_CK - 1) / ATT_CK;
    mh_f32x16 accv = {0}, acck = {0};
    fetch(0);
    for (int ch = 0; ch < chunks; ++ch) {
        __syncthreads();
        float pc[SPW], sc[SPW];
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            const int idx = tid + ATT_NT * i;
            abuf[(idx >> 6) * ATT_VP + (idx & 63)] = sa[i];
            qbuf[(idx >> 6) * ATT_VP + (idx & 63)] = sq[i];
        }
#pragma unroll
        for (int s = 0; s < SPW; ++s) {
            pc[s] = pf[s];
            sc[s] = sf[s];
        }
        __syncthreads();
        if (ch + 1 < chunks) fetch((ch + 1) * ATT_CK);
#pragma unroll
        for (int s = 0; s < SPW; ++s) {
            const int kk = 2 * (ks * SPW + s) + half;
            const float av = abuf[(db * 32 + l32) * ATT_VP + kk];
            const float aq = qbuf[(db * 32 + l32) * ATT_VP + kk];
            accv = __builtin_amdgcn_mfma_f32_32x32x2f32(av, pc[s], accv, 0, 0, 0);
            acck = __builtin_amdgcn_mfma_f32_32x32x2f32(aq, sc[s], acck, 0, 0, 0);
        }
    }
    float *outs[2] = {a.o0 + hoff, a.o1 + hoff};
#pragma unroll
    for (int which = 0; which < 2; ++which) {
        __syncthreads();
#pragma unroll
        for (int v = 0; v < 16; ++v)
            red[(wave * 32 + 8 * (v / 4) + 4 * half + (v % 4)) * ATT_RP + l32] = which ? acck[v] : accv[v];
        __syncthreads();
        for (int idx = tid; idx < HMAX * 32; idx += ATT_NT) {
            const int d = idx >> 5, cc = idx & 31;
            float s = 0.f;
#pragma unroll
            for (int k2 = 0; k2 < KS; ++k2) s += red[((k2 * DB + (d >> 5)) * 32 + (d & 31)) * ATT_RP + cc];
            if (d < H && c0 + cc < L) outs[which][(size_t)d * L + c0 + cc] = s;
        }
    }
}

// mat[b][f][l] += bias[f] for the three projections at once (mm_bias_add_transposed, per-row branch,
// lib/sources/pulp_train_utils_fp32.c:1286; lib/sources/pulp_mhsa_fp32.c:150-325).
__global__ __launch_bounds__(256) void mhsa_bias3_kernel(float *q, float *k, float *v, const float *bq,
                                                          const float *bk, const float *bv, size_t total, int F,
                                                          int L) {
    size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= total) return;
    const int f = (int)((idx / L) % F);
    float *m = blockIdx.y == 0 ? q : blockIdx.y == 1 ? k : v;
    const float *bias = blockIdx.y == 0 ? bq : blockIdx.y == 1 ? bk : bv;
    if (bias) m[idx] = m[idx] + bias[f];
}

// dx += tq + tk + tv in the reference's order (lib/sources/pulp_mhsa_fp32.c:1634-1745).
__global__ __launch_bounds__(256) void mhsa_sum3_kernel(float *dx, const float *t, size_t n) {
    size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= n) return;
    dx[idx] = ((dx[idx] + t[idx]) + t[n + idx]) + t[2 * n + idx];
}

// Row softmax over H rows of W (one wave per row).
__global__ __launch_bounds__(256) void softmax_fw_rows_kernel(const float *in, float *out, float *maxes,
                                                               float *sums, int H, int W) {
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (row >= H) return;
    const float *x = in + (size_t)row * W;
    float *y = out + (size_t)row * W;
    float mx = -FLT_MAX;
    for (int c = lane; c < W; c += 64) mx = fmaxf(mx, x[c]);
    mx = wave_max(mx);
    float sum = 0.f;
    for (int c = lane; c < W; c += 64) sum += fastexp_gist(x[c] - mx);
    sum = wave_sum(sum);
    for (int c = lane; c < W; c += 64) y[c] = fastexp_gist(x[c] - mx) / sum;
    if (lane == 0) {
        if (maxes) maxes[row] = mx;
        if (sums) sums[row] = sum;
    }
}

__global__ __launch_bounds__(256) void softmax_bw_rows_kernel(float *in_diff, const float *out, const float *out_diff,
                                                               float *sums, int H, int W) {
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (row >= H) return;
    const float *y = out + (size_t)row * W, *g = out_diff + (size_t)row * W;
    float sum = 0.f;
    for (int c = lane; c < W; c += 64) sum += g[c] * y[c];
    sum = wave_sum(sum);
    for (int c = lane; c < W; c += 64) in_diff[(size_t)row * W + c] = (g[c] - sum) * y[c];
    if (lane == 0 && sums) sums[row] = sum;
}

// ---------------------------------------------------------------------------------------------------------

struct MhsaDims {
    int L, E, F, heads, H;
};

static int mhsa_dims(const Mhsa_args *a, MhsaDims &m, const char *fn, bool backward) {
    auto bad = [&](const char *what) {
        printf("[%s] %s\n", fn, what);
        set_error("%s: %s", fn, what);
        return 1;
    };
    if (!a || !a->input || !a->output || !a->coeff_in_q || !a->coeff_in_k || !a->coeff_in_v || !a->coeff_out ||
        !a->q || !a->k || !a->v || !a->attention_map || !a->softmax_buffer)
        return bad("null argument structure");
    m.L = a->input->H;
    m.E = a->input->W;
    m.F = a->attention_map->W;
    m.heads = a->n_heads;
    if (m.L <= 0 || m.E <= 0 || m.F <= 0 || m.heads <= 0 || m.F % m.heads) return bad("invalid attention geometry");
    m.H = m.F / m.heads;
    if (m.H > 128) return bad("head size above 128 is not supported");
    if (m.L > 1024) return bad("sequence length above 1024 is not supported");
    const struct blob *act[] = {a->input, a->output, a->q, a->k, a->v, a->attention_map, a->softmax_buffer};
    for (const struct blob *bl : act)
        if (!bl->data || (backward && !bl->diff)) return bad("null activation buffer");
    const struct blob *wts[] = {a->coeff_in_q, a->coeff_in_k, a->coeff_in_v, a->coeff_out};
    for (const struct blob *bl : wts)
        if (!bl->data || (backward && !bl->diff)) return bad("null weight buffer");
    return 0;
}

static int att_lp(int L) { return ((L + ATT_CK - 1) / ATT_CK) * ATT_CK + 1; }

template <int HMAX>
static int launch_attn(int which, AttnArgs &a, int ns) {
    const size_t tile = (size_t)32 * a.LP, stage = (size_t)HMAX * ATT_VP, red = (size_t)4 * 32 * ATT_RP;
    const size_t lds = (which == 2 ? 2 * stage + red : tile + stage + red) * sizeof(float);
    void (*kern)(AttnArgs) =
        which == 0 ? attn_fw_kernel<HMAX> : which == 1 ? attn_bw_query_kernel<HMAX> : attn_bw_key_kernel<HMAX>;
    if (lds > 150 * 1024) {
        set_error("attention tile needs %zu bytes of LDS", lds);
        return 1;
    }
    static bool attr_set[3] = {false, false, false};
    if (!attr_set[which]) {
        if (!hip_ok(hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, 150 * 1024),
                    "hipFuncSetAttribute"))
            return 2;
        attr_set[which] = true;
    }
    dim3 grid((a.L + 31) / 32, a.heads, ns);
    hipLaunchKernelGGL(kern, grid, dim3(ATT_NT), lds, state().stream, a);
    return hip_ok(hipGetLastError(), "attention launch") ? 0 : 2;
}

static int launch_attn_any(int which, AttnArgs &a, int ns) {
    if (a.H <= 32) return launch_attn<32>(which, a, ns);
    if (a.H <= 64) return launch_attn<64>(which, a, ns);
    return launch_attn<128>(which, a, ns);
}

// C[b][n][l] = sum_k A(n,k) * B[b][k][l]: a weight matrix (element (n,k) at n*a_n + k*a_k) against a batch of
// [K][L] activations.
static int weight_times_acts(const float *A, int a_n, int a_k, const float *B, float *C, int N, int K, int L,
                             int ns) {
    GemmArgs g = {};
    g.a.HL = g.a.WL = g.b.HL = g.b.WL = 1;
    g.A = A;
    g.B = B;
    g.C = C;
    g.N = N;
    g.M = ns * L;
    g.K = K;
    g.a.row = axis_plain(N, a_n);
    g.a.k = axis_plain(K, a_k);
    g.b.row = axis_two(ns * L, L, K * L, 1);
    g.b.k = axis_plain(K, L);
    g.c.n = axis_plain(N, L);
    g.c.m = axis_two(ns * L, L, N * L, 1);
    return gemm<float>(g);
}

// C[n][m] = sum over samples and tokens of A[b][n][l] * B[b][m][l] (weight gradients).
static int acts_times_acts(const float *A, const float *B, float *C, int N, int M, int L, int ns) {
    GemmArgs g = {};
    g.a.HL = g.a.WL = g.b.HL = g.b.WL = 1;
    g.A = A;
    g.B = B;
    g.C = C;
    g.N = N;
    g.M = M;
    g.K = ns * L;
    g.a.row = axis_plain(N, L);
    g.a.k = axis_two(ns * L, L, N * L, 1);
    g.b.row = axis_plain(M, L);
    g.b.k = axis_two(ns * L, L, M * L, 1);
    g.c.n = axis_plain(N, M);
    g.c.m = axis_plain(M, 1);
    return gemm<float>(g);
}

static bool mhsa_fits(const MhsaDims &m, int ns) {
    const size_t lim = (size_t)1 << 31;
    return (size_t)ns * m.E * m.L < lim && (size_t)ns * m.F * m.L < lim && (size_t)ns * m.heads * m.L * m.L < lim &&
           (size_t)m.E * m.F < lim;
}

static int mhsa_fw(const Mhsa_args *a, int ns, const char *fn) {
    MhsaDims m;
    if (int rc = mhsa_dims(a, m, fn, false)) return rc;
    if (ns <= 0) return 0;
    if (!ensure_init()) return 2;
    if (!mhsa_fits(m, ns)) {
        set_error("%s: tensor larger than 2^31 elements", fn);
        return 1;
    }
    const int L = m.L, E = m.E, F = m.F;
    const size_t xe = (size_t)ns * E * L, fe = (size_t)ns * F * L, pe = (size_t)ns * m.heads * L * L;
    Stager sg;
    const float *X = sg.in(a->input->data, xe);
    const struct blob *wb[3] = {a->coeff_in_q, a->coeff_in_k, a->coeff_in_v};
    const struct blob *bb[3] = {a->bias_in_q, a->bias_in_k, a->bias_in_v};
    struct blob *ob[3] = {a->q, a->k, a->v};
    const float *W[3], *bias[3];
    float *QKV[3];
    for (int j = 0; j < 3; ++j) {
        W[j] = sg.in(wb[j]->data, (size_t)E * F);
        bias[j] = (bb[j] && bb[j]->data) ? sg.in(bb[j]->data, (size_t)F) : nullptr;
        QKV[j] = sg.out(ob[j]->data, fe);
    }
    const float *Wo = sg.in(a->coeff_out->data, (size_t)E * F);
    float *att = sg.out(a->attention_map->data, fe);
    float *P = sg.out(a->softmax_buffer->data, pe);
    float *Y = sg.out(a->output->data, xe);
    if (sg.failed()) return 2;
    int rc = 0;
    // q/k/v[F x L] = W^T . X + bias (weights stored E x F: lib/sources/pulp_mhsa_fp32.c:70-127)
    for (int j = 0; j < 3 && rc == 0; ++j) rc = weight_times_acts(W[j], 1, F, X, QKV[j], F, E, L, ns);
    if (rc == 0 && (bias[0] || bias[1] || bias[2])) {
        hipLaunchKernelGGL(mhsa_bias3_kernel, dim3((unsigned)((fe + 255) / 256), 3), dim3(256), 0, state().stream,
                           QKV[0], QKV[1], QKV[2], bias[0], bias[1], bias[2], fe, F, L);
        if (!hip_ok(hipGetLastError(), "bias launch")) rc = 2;
    }
    if (rc == 0) {
        AttnArgs t = {};
        t.q = QKV[0];
        t.k = QKV[1];
        t.v = QKV[2];
        t.o0 = P;
        t.o1 = att;
        t.L = L;
        t.H = m.H;
        t.heads = m.heads;
        t.F = F;
        t.LP = att_lp(L);
        t.scale = q_rsqrt_host((float)m.H);
        rc = launch_attn_any(0, t, ns);
    }
    // output[E x L] = Wout[E x F] . attention_map (:599-609)
    if (rc == 0) rc = weight_times_acts(Wo, F, 1, att, Y, E, F, L, ns);
    return sg.finish(rc);
}

static int mhsa_bw(const Mhsa_args *a, int ns, const char *fn) {
    MhsaDims m;
    if (int rc = mhsa_dims(a, m, fn, true)) return rc;
    if (ns <= 0) return 0;
    if (!ensure_init()) return 2;
    if (!mhsa_fits(m, ns)) {
        set_error("%s: tensor larger than 2^31 elements", fn);
        return 1;
    }
    const int L = m.L, E = m.E, F = m.F;
    const size_t xe = (size_t)ns * E * L, fe = (size_t)ns * F * L, pe = (size_t)ns * m.heads * L * L;
    const size_t rows = (size_t)ns * m.heads * L;
    Stager sg;
    const float *X = sg.in(a->input->data, xe);
    const float *dY = sg.in(a->output->diff, xe);
    float *dX = sg.inout(a->input->diff, xe);
    const struct blob *wb[3] = {a->coeff_in_q, a->coeff_in_k, a->coeff_in_v};
    struct blob *ob[3] = {a->q, a->k, a->v};
    const float *W[3], *QKV[3];
    float *dW[3], *dQKV[3];
    for (int j = 0; j < 3; ++j) {
        W[j] = sg.in(wb[j]->data, (size_t)E * F);
        dW[j] = sg.out(wb[j]->diff, (size_t)E * F);
        QKV[j] = sg.in(ob[j]->data, fe);
        dQKV[j] = sg.out(ob[j]->diff, fe);
    }
    const float *Wo = sg.in(a->coeff_out->data, (size_t)E * F);
    float *dWo = sg.out(a->coeff_out->diff, (size_t)E * F);
    const float *att = sg.in(a->attention_map->data, fe);
    float *datt = sg.out(a->attention_map->diff, fe);
    const float *P = sg.in(a->softmax_buffer->data, pe);
    float *dP = sg.out(a->softmax_buffer->diff, pe);
    if (sg.failed()) return 2;
    float *tmp = static_cast<float *>(scratch((3 * xe + rows) * sizeof(float)));
    if (!tmp) return 2;
    float *rs = tmp + 3 * xe;
    int rc = 0;
    // dWout[E x F] = dY . att^T (:742-760); datt[F x L] = Wout^T . dY (:816-834)
    rc = acts_times_acts(dY, att, dWo, E, F, L, ns);
    if (rc == 0) rc = weight_times_acts(Wo, 1, F, dY, datt, F, E, L, ns);
    AttnArgs t = {};
    t.q = QKV[0];
    t.k = QKV[1];
    t.v = QKV[2];
    t.p = P;
    t.da = datt;
    t.L = L;
    t.H = m.H;
    t.heads = m.heads;
    t.F = F;
    t.LP = att_lp(L);
    t.scale = q_rsqrt_host((float)m.H);
    if (rc == 0) {
        t.o0 = dP;
        t.o1 = dQKV[0];
        t.o2 = rs;
        rc = launch_attn_any(1, t, ns);
    }
    if (rc == 0) {
        t.dp = dP;
        t.rs = rs;
        t.o0 = dQKV[2];
        t.o1 = dQKV[1];
        t.o2 = nullptr;
        rc = launch_attn_any(2, t, ns);
    }
    for (int j = 0; j < 3 && rc == 0; ++j) {
        // dW[F x E] = d{q,k,v} . X^T (:1425-1560); temp[E x L] = W . d{q,k,v} (:1589-1744)
        rc = acts_times_acts(dQKV[j], X, dW[j], F, E, L, ns);
        if (rc == 0) rc = weight_times_acts(W[j], F, 1, dQKV[j], tmp + j * xe, E, F, L, ns);
    }
    if (rc == 0) {
        hipLaunchKernelGGL(mhsa_sum3_kernel, dim3((unsigned)((xe + 255) / 256)), dim3(256), 0, state().stream, dX,
                           tmp, xe);
        if (!hip_ok(hipGetLastError(), "sum launch")) rc = 2;
    }
    return sg.finish(rc);
}

static int softmax_rows(const softmax_args *a, bool backward, const char *fn) {
    if (!a || a->H <= 0 || a->W <= 0 || !a->output_data || (backward ? (!a->input_diff || !a->output_diff)
                                                                      : !a->input_data)) {
        printf("[%s] invalid arguments\n", fn);
        set_error("%s: invalid arguments", fn);
        return 1;
    }
    if (!ensure_init()) return 2;
    const size_t n = (size_t)a->H * a->W;
    Stager sg;
    dim3 grid((a->H + 3) / 4);
    if (!backward) {
        // the rows may be transformed in place (input == output): every element is read and written by one lane
        const float *in;
        float *out;
        if (a->output_data == a->input_data) {
            out = sg.inout(a->output_data, n);
            in = out;
        } else {
            in = sg.in(a->input_data, n);
            out = sg.out(a->output_data, n);
        }
        float *mx = a->maxes ? sg.out(a->maxes, (size_t)a->H) : nullptr;
        float *sm = a->sums ? sg.out(a->sums, (size_t)a->H) : nullptr;
        if (sg.failed()) return 2;
        hipLaunchKernelGGL(softmax_fw_rows_kernel, grid, dim3(256), 0, state().stream, in, out, mx, sm, a->H, a->W);
    } else {
        const float *y = sg.in(a->output_data, n);
        const float *g = sg.in(a->output_diff, n);
        float *gi = sg.out(a->input_diff, n);
        float *sm = a->sums ? sg.out(a->sums, (size_t)a->H) : nullptr;
        if (sg.failed()) return 2;
        hipLaunchKernelGGL(softmax_bw_rows_kernel, grid, dim3(256), 0, state().stream, gi, y, g, sm, a->H, a->W);
    }
    return sg.finish(hip_ok(hipGetLastError(), "softmax launch") ? 0 : 2);
}

}  // namespace ptl

extern "C" {

int ptl_mhsa_fp32_fw_batched(const struct Mhsa_args *a, int nsamples) {
    return ptl::mhsa_fw(a, nsamples, "pulp_mhsa_fp32_fw_cl");
}
int ptl_mhsa_fp32_bw_batched(const struct Mhsa_args *a, int nsamples) {
    return ptl::mhsa_bw(a, nsamples, "pulp_mhsa_fp32_bw_cl");
}
int ptl_internal_softmax_fp32(const struct softmax_args *a, int backward) {
    return ptl::softmax_rows(a, backward != 0, backward ? "pulp_softmax_fp32_bw_cl" : "pulp_softmax_fp32_fw_cl");
}

}  // extern "C"
