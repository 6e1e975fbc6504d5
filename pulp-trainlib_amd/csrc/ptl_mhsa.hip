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
#include "ptl_gemm_async.hpp"
#include "ptl_gemm_async.inc"
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

// ---------------------------------------------------------------------------------------------------------
// Tile loader: element (i, j), i < nrows, j < ncols (a multiple of 4), comes from g[i*gstride + j] when
// i < rvalid and j < cvalid and is zero otherwise; it lands at lds[i*pitch + j].  Each lane moves four
// consecutive columns with one 16-byte LDS-DMA load (global addresses need only 4-byte alignment, so rows of
// odd length are fine); a vector that straddles the end of a row is left to tile_edge_load/store, so
// nothing is ever read outside [0, rvalid) x [0, cvalid).  Two shapes: 32-column tiles stored with pitch 32
// (eight rows per instruction) and long rows (up to 256 columns per instruction, any pitch that is a multiple
// of 4).  Work is dealt to the NW waves of the workgroup; completion = the caller's vmcnt wait + barrier.
template <int NW>
__device__ inline void tile_dma(const float *__restrict__ g, long long gstride, int nrows, int ncols, int rvalid,
                                int cvalid, float *lds, int pitch, const float *zero, int wave, int lane) {
    const unsigned lds_addr = (unsigned)(uintptr_t)(lds_char *)lds;
    int ninstr, rows_per, lanes_per_row, segs;
    if (ncols == 32 && pitch == 32) {
        rows_per = 8;
        lanes_per_row = 8;
        segs = 1;
        ninstr = (nrows + 7) >> 3;
    } else {
        rows_per = 1;
        lanes_per_row = 64;
        segs = (ncols + 255) >> 8;
        ninstr = nrows * segs;
    }
    for (int j = wave; j < ninstr; j += NW) {
        int i, col;
        unsigned m0;
        if (rows_per == 8) {
            i = j * 8 + (lane >> 3);
            col = (lane & 7) * 4;
            m0 = lds_addr + (unsigned)j * 1024u;
        } else {
            const int seg = j % segs;
            i = j / segs;
            col = seg * 256 + lane * 4;
            m0 = lds_addr + ((unsigned)i * pitch + seg * 256) * 4u;
        }
        if (i >= nrows || col >= ncols) continue;
        const bool row_ok = i < rvalid;
        const bool full = row_ok && col + 4 <= cvalid;
        if (row_ok && !full && col < cvalid) continue;  // straddles the end of the row: second pass
        lds_dma<16>(full ? g + (long long)i * gstride + col : zero, m0);
    }
}

// The vector of a tile row that straddles the end of the valid columns (at most one per row): thread `tid`
// of the workgroup loads the one of row `tid` with element loads, and stores it once every tile of the volley
// has been enqueued, so that all these loads are in flight together.  Tiles have at most 256 rows.
struct TileEdge {
    float4 v;
    float *dst;
};

__device__ inline TileEdge tile_edge_load(const float *__restrict__ g, long long gstride, int nrows, int ncols,
                                          int rvalid, int cvalid, float *lds, int pitch, int tid) {
    TileEdge e;
    e.dst = nullptr;
    e.v = make_float4(0.f, 0.f, 0.f, 0.f);
    const int pcol = cvalid & ~3;
    if ((cvalid & 3) && pcol < ncols && tid < nrows && tid < rvalid) {
        const float *src = g + (long long)tid * gstride + pcol;
        e.v.x = src[0];
        if (pcol + 1 < cvalid) e.v.y = src[1];
        if (pcol + 2 < cvalid) e.v.z = src[2];
        e.dst = lds + (size_t)tid * pitch + pcol;
    }
    return e;
}

__device__ inline void tile_edge_store(const TileEdge &e) {
    if (e.dst) *reinterpret_cast<float4 *>(e.dst) = e.v;
}

// ---------------------------------------------------------------------------------------------------------
// Panel product for the projections and their gradients.
//
//   C[n][m] (+)= bias[n] + sum over terms t, samples b (gradient mode) and k of A_t(n,k) * B_t(m,k)
//
// where A_t(n,k) sits at A_t + b*a_s + n*a_n + k*a_k (B alike) and one of the two strides of each operand
// is 1.  The whole 32-row x <=200-deep panel of each operand goes from global memory to LDS in one volley of
// LDS-DMA loads, all in flight together: one trip to memory per panel.  The four waves split the contraction
// in groups of eight k and meet in LDS.  LDS layouts: [k][32 rows] when rows are contiguous in memory
// (fragment = four 4-byte reads, lanes along rows), [row][k] with a pitch of 204 floats (an odd number of
// 16-byte units) when k is (fragment = one 16-byte read); both are free of bank conflicts.
constexpr int PG_KC = 200;          // contraction depth of a panel (multiple of 8)
constexpr int PG_P = PG_KC + 4;     // pitch of the [row][k] layout
constexpr int PG_PANEL = 32 * PG_P; // floats per operand panel (the [k][32] layout needs 32 * PG_KC)

struct PanelArgs {
    const float *A[3], *B[3];  // operands of term t (fan-in) or output o (fan-out)
    float *C[3];
    const float *bias[3];
    const float *zero;         // source of elements that do not exist
    float *part;               // partial sums [nout][groups][N][M] when groups > 1
    int nout, nterm;
    int N, M, K;
    int a_n, a_k, b_m, b_k;
    long long a_s, b_s, c_s;   // per-sample element strides
    int c_n;                   // output row stride (columns contiguous)
    int ns;
    int sum_samples;           // 1: the contraction also runs over the samples (weight gradients)
    int spg, groups;           // samples per workgroup and number of sample groups in that mode
    int accumulate;            // 1: add to what C holds
};

// Panel of rows [r0, r0+32) x k [k0, k0+PG_KC) of an operand with row stride s_r and k stride s_k.
template <bool KMAJ, int NW>
__device__ inline TileEdge panel_load(const float *g, int s_r, int s_k, int r0, int R, int k0, int K, float *lds,
                                      const float *zero, int tid, int wave, int lane) {
    if (KMAJ) {
        const float *t = g + (long long)r0 * s_r + k0;
        tile_dma<NW>(t, s_r, 32, PG_KC, R - r0, K - k0, lds, PG_P, zero, wave, lane);
        return tile_edge_load(t, s_r, 32, PG_KC, R - r0, K - k0, lds, PG_P, tid);
    }
    const float *t = g + (long long)k0 * s_k + r0;
    tile_dma<NW>(t, s_k, PG_KC, 32, K - k0, R - r0, lds, 32, zero, wave, lane);
    return tile_edge_load(t, s_k, PG_KC, 32, K - k0, R - r0, lds, 32, tid);
}

// The four k values [k4, k4+4) of row r.
template <bool KMAJ>
__device__ inline float4 panel_frag(const float *lds, int r, int k4) {
    if (KMAJ) return *reinterpret_cast<const float4 *>(lds + r * PG_P + k4);
    float4 v;
    v.x = lds[k4 * 32 + r];
    v.y = lds[(k4 + 1) * 32 + r];
    v.z = lds[(k4 + 2) * 32 + r];
    v.w = lds[(k4 + 3) * 32 + r];
    return v;
}

__device__ inline void mfma4(mh_f32x16 &acc, const float4 &a, const float4 &b) {
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.x, b.x, acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.y, b.y, acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.z, b.z, acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.w, b.w, acc, 0, 0, 0);
}

// NB row blocks of 32 per workgroup share one B panel; each block has its own four waves.  (bx, by, bz): the
// workgroup's place in the product's grid of (column blocks, row blocks, outputs x samples or sample groups).
template <bool A_KMAJ, bool B_KMAJ, int NB>
__device__ __forceinline__ void panel_gemm_body(const PanelArgs &a, unsigned bx, unsigned by, unsigned bz) {
    extern __shared__ __attribute__((aligned(16))) float pg_lds[];
    constexpr int NW = 4 * NB, NT = ATT_NT * NB;
    float *Bs = pg_lds, *As = pg_lds + PG_PANEL;  // As: NB panels
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31, half = lane >> 5;
    const int nb = wave >> 2, ks = wave & 3;
    const int m0 = (int)bx * 32, n0 = (int)by * (32 * NB);
    int o, b_first, b_count, grp = 0;
    if (a.sum_samples) {
        o = (int)bz / a.groups;
        grp = (int)bz % a.groups;
        b_first = grp * a.spg;
        b_count = min(a.spg, a.ns - b_first);
    } else {
        o = (int)bz / a.ns;
        b_first = (int)bz % a.ns;
        b_count = 1;
    }
    mh_f32x16 acc = {0};
    for (int bi = 0; bi < b_count; ++bi)
        for (int t = 0; t < a.nterm; ++t) {
            const float *Ag = a.A[o * a.nterm + t] + (long long)(b_first + bi) * a.a_s;
            const float *Bg = a.B[o * a.nterm + t] + (long long)(b_first + bi) * a.b_s;
            for (int k0 = 0; k0 < a.K; k0 += PG_KC) {
                __syncthreads();  // the previous panels have been consumed
                TileEdge ea[NB];
#pragma unroll
                for (int j = 0; j < NB; ++j) {
                    ea[j].dst = nullptr;
                    if (n0 + 32 * j < a.N)
                        ea[j] = panel_load<A_KMAJ, NW>(Ag, a.a_n, a.a_k, n0 + 32 * j, a.N, k0, a.K, As + j * PG_PANEL,
                                                       a.zero, tid, wave, lane);
                }
                const TileEdge eb = panel_load<B_KMAJ, NW>(Bg, a.b_m, a.b_k, m0, a.M, k0, a.K, Bs, a.zero, tid, wave,
                                                           lane);
#pragma unroll
                for (int j = 0; j < NB; ++j) tile_edge_store(ea[j]);
                tile_edge_store(eb);
                wait_vmcnt<0>();
                __syncthreads();
                // groups of eight k (beyond the valid depth the panels hold zeros), dealt to the four waves of a
                // row block in runs; within a group the lower half-wave takes k 0..3 and the upper 4..7
                if (n0 + 32 * nb < a.N) {
                    const float *Aw = As + nb * PG_PANEL;
                    const int ngroups = (min(PG_KC, a.K - k0) + 7) >> 3;
                    const int per = (ngroups + 3) >> 2;
                    const int g_end = min(ngroups, (ks + 1) * per);
                    for (int gq = ks * per; gq < g_end; ++gq) {
                        const int k4 = gq * 8 + half * 4;
                        mfma4(acc, panel_frag<A_KMAJ>(Aw, l32, k4), panel_frag<B_KMAJ>(Bs, l32, k4));
                    }
                }
            }
        }
    __syncthreads();
    float *red = pg_lds;
#pragma unroll
    for (int v = 0; v < 16; ++v) red[(wave * 32 + 8 * (v / 4) + 4 * half + (v % 4)) * ATT_RP + l32] = acc[v];
    __syncthreads();
    const bool partial = a.sum_samples && a.groups > 1;
    float *Cb = partial ? a.part + ((size_t)o * a.groups + grp) * a.N * a.M
                        : a.C[o] + (a.sum_samples ? 0 : (long long)b_first * a.c_s);
    const int c_n = partial ? a.M : a.c_n;
    const float *bias = partial ? nullptr : a.bias[o];
    for (int idx = tid; idx < 1024 * NB; idx += NT) {
        const int n = idx >> 5, m = idx & 31;  // n in [0, 32*NB)
        const float *r = red + ((n >> 5) * 128 + (n & 31)) * ATT_RP + m;
        float v = ((r[0] + r[32 * ATT_RP]) + r[64 * ATT_RP]) + r[96 * ATT_RP];
        if (n0 + n < a.N && m0 + m < a.M) {
            float *dst = Cb + (size_t)(n0 + n) * c_n + m0 + m;
            if (bias) v = v + bias[n0 + n];
            if (a.accumulate && !partial) v = *dst + v;
            *dst = v;
        }
    }
}

template <bool A_KMAJ, bool B_KMAJ, int NB>
__global__ __launch_bounds__(ATT_NT * NB) void panel_gemm_kernel(PanelArgs a) {
    panel_gemm_body<A_KMAJ, B_KMAJ, NB>(a, blockIdx.x, blockIdx.y, blockIdx.z);
}

// Two independent products in one launch (both read what the launch before them wrote, neither reads the other):
// the first n0 workgroups are the first product's grid (gx0 x gy0 x gz0, x fastest), the rest the second's.  The
// block is as large as the larger of the two needs; the waves a product does not use leave at once.
struct PanelPairGrid {
    unsigned n0, gx0, gy0, gx1, gy1;
    int nb0, nb1;
};

template <bool AK0, bool BK0, bool AK1, bool BK1>
__global__ __launch_bounds__(ATT_NT * 2) void panel_gemm_pair_kernel(PanelArgs a, PanelArgs b, PanelPairGrid g) {
    unsigned id = blockIdx.x;
    if (id < g.n0) {
        if ((int)threadIdx.x >= ATT_NT * g.nb0) return;
        const unsigned bx = id % g.gx0, r = id / g.gx0;
        if (g.nb0 == 2)
            panel_gemm_body<AK0, BK0, 2>(a, bx, r % g.gy0, r / g.gy0);
        else
            panel_gemm_body<AK0, BK0, 1>(a, bx, r % g.gy0, r / g.gy0);
    } else {
        id -= g.n0;
        if ((int)threadIdx.x >= ATT_NT * g.nb1) return;
        const unsigned bx = id % g.gx1, r = id / g.gx1;
        if (g.nb1 == 2)
            panel_gemm_body<AK1, BK1, 2>(b, bx, r % g.gy1, r / g.gy1);
        else
            panel_gemm_body<AK1, BK1, 1>(b, bx, r % g.gy1, r / g.gy1);
    }
}

// C_o[i] = sum over groups of part[o][g][i]   (+ what C holds when accumulate)
__device__ __forceinline__ void panel_reduce_body(const PanelArgs &a, int o) {
    const size_t nm = (size_t)a.N * a.M, i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= nm) return;
    const float *p = a.part + (size_t)o * a.groups * nm + i;
    // eight loads in flight at a time (a serial walk is one trip to memory per group); the sums are added in
    // the order of the groups either way
    float s = 0.f;
    int g = 0;
    for (; g + 8 <= a.groups; g += 8) {
        float v[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = p[(size_t)(g + j) * nm];
#pragma unroll
        for (int j = 0; j < 8; ++j) s += v[j];
    }
    for (; g < a.groups; ++g) s += p[(size_t)g * nm];
    float *dst = a.C[o] + (i / a.M) * a.c_n + (i % a.M);
    *dst = a.accumulate ? *dst + s : s;
}

__global__ __launch_bounds__(256) void panel_reduce_kernel(PanelArgs a) { panel_reduce_body(a, blockIdx.y); }

// ... of two products at once: blockIdx.y runs over the outputs of the first, then of the second
__global__ __launch_bounds__(256) void panel_reduce_pair_kernel(PanelArgs a, PanelArgs b) {
    if ((int)blockIdx.y < a.nout)
        panel_reduce_body(a, blockIdx.y);
    else
        panel_reduce_body(b, (int)blockIdx.y - a.nout);
}

struct AttnArgs {
    const float *q, *k, *v;  // [ns][F][L]
    const float *p;          // probabilities [ns][heads][L][L]   (backward)
    const float *da;         // attention_map gradient [ns][F][L]  (backward)
    const float *dp;         // probability gradient               (backward II)
    const float *rs;         // row sums of dP.P [ns][heads][L]    (backward II)
    float *o0, *o1, *o2;     // kernel outputs (see each kernel)
    const float *zero;       // 256 zero bytes: source of elements that do not exist
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

// ---------------------------------------------------------------------------------------------------------
// Resident variants for sequences of at most 200 tokens and head sizes of 33..64 (ViT geometry): everything a
// workgroup needs comes in by LDS-DMA in one volley at its start (a single trip to memory instead of one per
// phase), and all fragments are read from LDS.  Sixteen waves per workgroup (one workgroup per CU: the panels
// take 150 KB), so that every SIMD has four waves to choose from while some wait (measured 3 % faster than eight).
constexpr int RS_NW = 16;           // waves
constexpr int RS_NT = RS_NW * 64;   // threads
constexpr int RS_RPW = 32 / RS_NW;  // score rows per wave
constexpr int RS_KS = RS_NW / 2;    // contraction ranges of the token-contracting products
constexpr int RS_LC = 224;  // key columns covered: 7 blocks of 32
constexpr int RS_KD = 200;  // contraction depth over tokens (25 groups of 8)
constexpr int RS_KP = 232;  // pitch of a [d][token] panel read with lanes along tokens (4 rows apart = 32 banks)
constexpr int RS_VP = 204;  // pitch of a [d][token] panel read as 16-byte fragments along tokens
constexpr int RS_SP = 228;  // pitch of the [32][token] score tile (16-byte fragments along tokens)
constexpr int RS_FW_FLOATS = 64 * 32 + 64 * RS_KP + 64 * RS_VP + 32 * RS_SP;
constexpr int RS_KEY_FLOATS = 2 * 64 * RS_VP + 2 * RS_KD * 32 + RS_KD;
static_assert(RS_NW * 32 * ATT_RP <= 64 * 32 + 64 * RS_KP, "parked accumulators fit the first two panels");

// S[r][c] = scale * sum_d Rs[d][r] * Cs[d][c]: Rs is [64][32], Cs [64][RS_KP], both in LDS; one 32-column
// block per wave.
__device__ inline void scores_resident(const float *Rs, const float *Cs, int CB, float scale, float *S, int wave,
                                       int l32, int half) {
    for (int cb = wave; cb < CB; cb += RS_NW) {
        mh_f32x16 acc = {0};
#pragma unroll
        for (int g = 0; g < 8; ++g) {
            const int d4 = g * 8 + half * 4;
            float4 x, y;
            x.x = Rs[d4 * 32 + l32];
            x.y = Rs[(d4 + 1) * 32 + l32];
            x.z = Rs[(d4 + 2) * 32 + l32];
            x.w = Rs[(d4 + 3) * 32 + l32];
            const float *cp = Cs + d4 * RS_KP + cb * 32 + l32;
            y.x = cp[0];
            y.y = cp[RS_KP];
            y.z = cp[2 * RS_KP];
            y.w = cp[3 * RS_KP];
            mfma4(acc, x, y);
        }
#pragma unroll
        for (int v = 0; v < 16; ++v) S[(8 * (v / 4) + 4 * half + (v % 4)) * RS_SP + cb * 32 + l32] = acc[v] * scale;
    }
}

// Parked partial tiles of the RS_KS contraction ranges -> out[d][x0 + x] (d < H, x0 + x < L).
__device__ inline void mix_store(const float *red, int L, int H, int x0, float *__restrict__ out, int tid) {
    for (int idx = tid; idx < 64 * 32; idx += RS_NT) {
        const int d = idx >> 5, xx = idx & 31;
        float s = 0.f;
#pragma unroll
        for (int k2 = 0; k2 < RS_KS; ++k2) s += red[((2 * k2 + (d >> 5)) * 32 + (d & 31)) * ATT_RP + xx];
        if (d < H && x0 + xx < L) out[(size_t)d * L + x0 + xx] = s;
    }
}

// out[d][r0 + r] = sum_c Vs[d][c] * S[r][c] (d < H): Vs [64][RS_VP] and S [32][RS_SP] in LDS, S zero beyond L.
// Waves: (block of 32 d) x (range of the contraction); the ranges meet in `red`.
__device__ inline void mix_resident(const float *Vs, const float *S, int L, int H, int r0, float *__restrict__ out,
                                    float *red, int tid, int wave, int l32, int half) {
    const int db = wave & 1, ks = wave >> 1;
    const int ngroups = (L + 7) >> 3, per = (ngroups + RS_KS - 1) / RS_KS;
    const int g_end = min(ngroups, (ks + 1) * per);
    mh_f32x16 acc = {0};
    for (int g = ks * per; g < g_end; ++g) {
        const int k4 = g * 8 + half * 4;
        mfma4(acc, *reinterpret_cast<const float4 *>(Vs + (db * 32 + l32) * RS_VP + k4),
              *reinterpret_cast<const float4 *>(S + l32 * RS_SP + k4));
    }
#pragma unroll
    for (int v = 0; v < 16; ++v) red[(wave * 32 + 8 * (v / 4) + 4 * half + (v % 4)) * ATT_RP + l32] = acc[v];
    __syncthreads();
    mix_store(red, L, H, r0, out, tid);
}

__global__ __launch_bounds__(RS_NT) void attn_fw_res_kernel(AttnArgs a) {
    extern __shared__ __attribute__((aligned(16))) float att_lds[];
    float *Qs = att_lds, *Ks = Qs + 64 * 32, *Vs = Ks + 64 * RS_KP, *S = Vs + 64 * RS_VP, *red = att_lds;
    const int r0 = blockIdx.x * 32, h = blockIdx.y, b = blockIdx.z, L = a.L;
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31, half = lane >> 5;
    const size_t hoff = ((size_t)b * a.F + (size_t)h * a.H) * L;
    tile_dma<RS_NW>(a.q + hoff + r0, L, 64, 32, a.H, L - r0, Qs, 32, a.zero, wave, lane);
    tile_dma<RS_NW>(a.k + hoff, L, 64, RS_LC, a.H, L, Ks, RS_KP, a.zero, wave, lane);
    tile_dma<RS_NW>(a.v + hoff, L, 64, RS_KD, a.H, L, Vs, RS_VP, a.zero, wave, lane);
    const TileEdge e0 = tile_edge_load(a.q + hoff + r0, L, 64, 32, a.H, L - r0, Qs, 32, tid);
    const TileEdge e1 = tile_edge_load(a.k + hoff, L, 64, RS_LC, a.H, L, Ks, RS_KP, tid);
    const TileEdge e2 = tile_edge_load(a.v + hoff, L, 64, RS_KD, a.H, L, Vs, RS_VP, tid);
    tile_edge_store(e0);
    tile_edge_store(e1);
    tile_edge_store(e2);
    wait_vmcnt<0>();
    __syncthreads();
    scores_resident(Qs, Ks, (L + 31) >> 5, a.scale, S, wave, l32, half);
    __syncthreads();
    // softmax of this wave's rows over the keys (lib/sources/pulp_act_fp32.c:187-225): max, approximate
    // exponential of the difference, sum, division; the rows' reductions run side by side
    float *P = a.o0 + ((size_t)b * a.heads + h) * L * L;
    float sv[RS_RPW][4], mx[RS_RPW], sum[RS_RPW];
#pragma unroll
    for (int i = 0; i < RS_RPW; ++i) {
        const float *srow = S + (wave * RS_RPW + i) * RS_SP;
        mx[i] = -FLT_MAX;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int c = lane + 64 * j;
            sv[i][j] = c < L ? srow[c] : -FLT_MAX;
            mx[i] = fmaxf(mx[i], sv[i][j]);
        }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1)
#pragma unroll
        for (int i = 0; i < RS_RPW; ++i) mx[i] = fmaxf(mx[i], __shfl_xor(mx[i], o));
#pragma unroll
    for (int i = 0; i < RS_RPW; ++i) {
        sum[i] = 0.f;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int c = lane + 64 * j;
            sv[i][j] = c < L ? fastexp_gist(sv[i][j] - mx[i]) : 0.f;
            sum[i] += sv[i][j];
        }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1)
#pragma unroll
        for (int i = 0; i < RS_RPW; ++i) sum[i] += __shfl_xor(sum[i], o);
#pragma unroll
    for (int i = 0; i < RS_RPW; ++i) {
        const int row = wave * RS_RPW + i;
        float *srow = S + row * RS_SP;
        const bool live = r0 + row < L;
        const float inv = 1.0f / sum[i];  // one division per row; the products differ from quotients by an ulp at most
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int c = lane + 64 * j;
            if (c < RS_LC) {
                const float pv = c < L ? sv[i][j] * inv : 0.f;
                srow[c] = pv;
                if (live && c < L) P[(size_t)(r0 + row) * L + c] = pv;
            }
        }
    }
    __syncthreads();
    mix_resident(Vs, S, L, a.H, r0, a.o1 + hoff, red, tid, wave, l32, half);
}

__global__ __launch_bounds__(RS_NT) void attn_bw_query_res_kernel(AttnArgs a) {
    extern __shared__ __attribute__((aligned(16))) float att_lds[];
    float *Qs = att_lds, *Ks = Qs + 64 * 32, *Vs = Ks + 64 * RS_KP, *S = Vs + 64 * RS_VP, *red = att_lds;
    const int r0 = blockIdx.x * 32, h = blockIdx.y, b = blockIdx.z, L = a.L;
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31, half = lane >> 5;
    const size_t hoff = ((size_t)b * a.F + (size_t)h * a.H) * L;
    const size_t poff = ((size_t)b * a.heads + h) * L * L;
    tile_dma<RS_NW>(a.da + hoff + r0, L, 64, 32, a.H, L - r0, Qs, 32, a.zero, wave, lane);
    tile_dma<RS_NW>(a.v + hoff, L, 64, RS_LC, a.H, L, Ks, RS_KP, a.zero, wave, lane);
    tile_dma<RS_NW>(a.k + hoff, L, 64, RS_KD, a.H, L, Vs, RS_VP, a.zero, wave, lane);
    const TileEdge e0 = tile_edge_load(a.da + hoff + r0, L, 64, 32, a.H, L - r0, Qs, 32, tid);
    const TileEdge e1 = tile_edge_load(a.v + hoff, L, 64, RS_LC, a.H, L, Ks, RS_KP, tid);
    const TileEdge e2 = tile_edge_load(a.k + hoff, L, 64, RS_KD, a.H, L, Vs, RS_VP, tid);
    // this wave's probability rows ride along in registers
    float pr[RS_RPW][4];
#pragma unroll
    for (int i = 0; i < RS_RPW; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int row = r0 + wave * RS_RPW + i, c = lane + 64 * j;
            pr[i][j] = (row < L && c < L) ? a.p[poff + (size_t)row * L + c] : 0.f;
        }
    tile_edge_store(e0);
    tile_edge_store(e1);
    tile_edge_store(e2);
    wait_vmcnt<0>();
    __syncthreads();
    // dP[query][key] = sum_d dA[d][query] v[d][key]   (lib/sources/pulp_mhsa_fp32.c:958-1060)
    scores_resident(Qs, Ks, (L + 31) >> 5, 1.0f, S, wave, l32, half);
    __syncthreads();
    // softmax backward (lib/sources/pulp_act_fp32.c:335-390) and the scaling (:1176-1183)
    float gv[RS_RPW][4], sum[RS_RPW];
#pragma unroll
    for (int i = 0; i < RS_RPW; ++i) {
        const float *srow = S + (wave * RS_RPW + i) * RS_SP;
        sum[i] = 0.f;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int c = lane + 64 * j;
            gv[i][j] = c < L ? srow[c] : 0.f;
            sum[i] += gv[i][j] * pr[i][j];
        }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1)
#pragma unroll
        for (int i = 0; i < RS_RPW; ++i) sum[i] += __shfl_xor(sum[i], o);
#pragma unroll
    for (int i = 0; i < RS_RPW; ++i) {
        const int row = wave * RS_RPW + i;
        float *srow = S + row * RS_SP;
        const bool live = r0 + row < L;
        float *dprow = a.o0 + poff + (size_t)(r0 + row) * L;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int c = lane + 64 * j;
            if (c < RS_LC) {
                if (live && c < L) dprow[c] = gv[i][j];
                srow[c] = c < L ? ((gv[i][j] - sum[i]) * pr[i][j]) * a.scale : 0.f;
            }
        }
        if (live && lane == 0) a.o2[((size_t)b * a.heads + h) * L + r0 + row] = sum[i];
    }
    __syncthreads();
    // dq[d][query] = sum_key k[d][key] dS[query][key]   (:1342-1360)
    mix_resident(Vs, S, L, a.H, r0, a.o1 + hoff, red, tid, wave, l32, half);
}

// Key side: tile of 32 keys; dA and q ([d][query], 16-byte fragments along the queries) and the key columns
// of P and dP ([query][32 keys]) are resident; dS replaces dP in place before the products.
//   dv[d][key] = sum_query dA[d][query] P[query][key]                         (:884-902)
//   dk[d][key] = sum_query q[d][query] dS[query][key], dS = (dP - rs) P scale  (:1244-1330)
__global__ __launch_bounds__(RS_NT) void attn_bw_key_res_kernel(AttnArgs a) {
    extern __shared__ __attribute__((aligned(16))) float att_lds[];
    float *dAs = att_lds, *Qs = dAs + 64 * RS_VP, *Pp = Qs + 64 * RS_VP, *Gp = Pp + RS_KD * 32, *rsl = Gp + RS_KD * 32;
    float *red = att_lds;
    const int c0 = blockIdx.x * 32, h = blockIdx.y, b = blockIdx.z, L = a.L, H = a.H;
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31, half = lane >> 5;
    const size_t hoff = ((size_t)b * a.F + (size_t)h * H) * L;
    const size_t poff = ((size_t)b * a.heads + h) * L * L;
    tile_dma<RS_NW>(a.da + hoff, L, 64, RS_KD, H, L, dAs, RS_VP, a.zero, wave, lane);
    tile_dma<RS_NW>(a.q + hoff, L, 64, RS_KD, H, L, Qs, RS_VP, a.zero, wave, lane);
    tile_dma<RS_NW>(a.p + poff + c0, L, RS_KD, 32, L, L - c0, Pp, 32, a.zero, wave, lane);
    tile_dma<RS_NW>(a.dp + poff + c0, L, RS_KD, 32, L, L - c0, Gp, 32, a.zero, wave, lane);
    const TileEdge e0 = tile_edge_load(a.da + hoff, L, 64, RS_KD, H, L, dAs, RS_VP, tid);
    const TileEdge e1 = tile_edge_load(a.q + hoff, L, 64, RS_KD, H, L, Qs, RS_VP, tid);
    const TileEdge e2 = tile_edge_load(a.p + poff + c0, L, RS_KD, 32, L, L - c0, Pp, 32, tid);
    const TileEdge e3 = tile_edge_load(a.dp + poff + c0, L, RS_KD, 32, L, L - c0, Gp, 32, tid);
    const float rsv = (tid < RS_KD && tid < L) ? a.rs[((size_t)b * a.heads + h) * L + tid] : 0.f;
    tile_edge_store(e0);
    tile_edge_store(e1);
    tile_edge_store(e2);
    tile_edge_store(e3);
    if (tid < RS_KD) rsl[tid] = rsv;
    wait_vmcnt<0>();
    __syncthreads();
    for (int idx = tid; idx < RS_KD * 32; idx += RS_NT) Gp[idx] = ((Gp[idx] - rsl[idx >> 5]) * Pp[idx]) * a.scale;
    __syncthreads();
    const int db = wave & 1, ks = wave >> 1;
    const int ngroups = (L + 7) >> 3, per = (ngroups + RS_KS - 1) / RS_KS;
    const int g_end = min(ngroups, (ks + 1) * per);
    mh_f32x16 accv = {0}, acck = {0};
    for (int g = ks * per; g < g_end; ++g) {
        const int k4 = g * 8 + half * 4;
        float4 pb, sb;
        pb.x = Pp[k4 * 32 + l32];
        pb.y = Pp[(k4 + 1) * 32 + l32];
        pb.z = Pp[(k4 + 2) * 32 + l32];
        pb.w = Pp[(k4 + 3) * 32 + l32];
        sb.x = Gp[k4 * 32 + l32];
        sb.y = Gp[(k4 + 1) * 32 + l32];
        sb.z = Gp[(k4 + 2) * 32 + l32];
        sb.w = Gp[(k4 + 3) * 32 + l32];
        mfma4(accv, *reinterpret_cast<const float4 *>(dAs + (db * 32 + l32) * RS_VP + k4), pb);
        mfma4(acck, *reinterpret_cast<const float4 *>(Qs + (db * 32 + l32) * RS_VP + k4), sb);
    }
    float *outs[2] = {a.o0 + hoff, a.o1 + hoff};
#pragma unroll
    for (int which = 0; which < 2; ++which) {
        __syncthreads();
#pragma unroll
        for (int v = 0; v < 16; ++v)
            red[(wave * 32 + 8 * (v / 4) + 4 * half + (v % 4)) * ATT_RP + l32] = which ? acck[v] : accv[v];
        __syncthreads();
        mix_store(red, L, H, c0, outs[which], tid);
    }
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
    if (a.L <= RS_KD && a.H > 32 && a.H <= 64) {
        a.zero = static_cast<const float *>(state().zeros);
        if (!a.zero) return 2;
        void (*kern)(AttnArgs) =
            which == 0 ? attn_fw_res_kernel : which == 1 ? attn_bw_query_res_kernel : attn_bw_key_res_kernel;
        const size_t lds = (size_t)(which == 2 ? RS_KEY_FLOATS : RS_FW_FLOATS) * sizeof(float);
        static bool attr_set[3] = {false, false, false};
        if (!attr_set[which]) {
            if (!hip_ok(hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                            hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024),
                        "hipFuncSetAttribute"))
                return 2;
            attr_set[which] = true;
        }
        dim3 grid((a.L + 31) / 32, a.heads, ns);
        hipLaunchKernelGGL(kern, grid, dim3(RS_NT), lds, state().stream, a);
        return hip_ok(hipGetLastError(), "attention launch") ? 0 : 2;
    }
    if (a.H <= 32) return launch_attn<32>(which, a, ns);
    if (a.H <= 64) return launch_attn<64>(which, a, ns);
    return launch_attn<128>(which, a, ns);
}

// Sample groups the gradient mode of the panel product uses for `nout` N x M outputs: enough workgroups to
// fill the chip a few times over.
static int panel_groups(int nout, int N, int M, int ns) {
    const long tiles = (long)((N + 31) / 32) * ((M + 31) / 32) * nout;
    long groups = (4L * state().num_cu + tiles - 1) / tiles;
    if (groups > ns) groups = ns;
    return groups < 1 ? 1 : (int)groups;
}

static size_t panel_part_floats(int nout, int N, int M, int ns) {
    const int g = panel_groups(nout, N, M, ns);
    return g > 1 ? (size_t)nout * g * N * M : 0;
}

// Launches the panel product; `p` carries operands, strides and sizes, this fills in the rest.  In gradient
// mode (sum_samples) the partial sums of the sample groups go to `part` and a second kernel adds them.
// What a launch of the panel product needs besides its arguments.
struct PanelPlan {
    bool ak, bk;
    int nb;
    dim3 grid;
    size_t lds;
};

// Fills in the fields of `p` the caller leaves open (zero page, sample groups, partial sums) and works out the
// launch.  0, or the error code.
static int panel_plan(PanelArgs &p, float *part, PanelPlan &pl) {
    State &st = state();
    p.zero = static_cast<const float *>(st.zeros);
    if (!p.zero) return 2;
    if ((p.a_k != 1 && p.a_n != 1) || (p.b_k != 1 && p.b_m != 1)) {
        set_error("panel product: operand without a unit stride");
        return 1;
    }
    pl.ak = p.a_k == 1;
    pl.bk = p.b_k == 1;
    p.groups = 1;
    p.spg = p.ns;
    p.part = nullptr;
    if (p.sum_samples) {
        const int groups = panel_groups(p.nout, p.N, p.M, p.ns);
        if (groups > 1) {
            p.spg = (p.ns + groups - 1) / groups;
            p.groups = (p.ns + p.spg - 1) / p.spg;
            p.part = part;
            if (!part) return 2;
        }
    }
    // Two row blocks per workgroup (the B panel is fetched once for both) when single blocks would already
    // queue up behind each other on the CUs.
    const size_t zdim = p.sum_samples ? (size_t)p.nout * p.groups : (size_t)p.nout * p.ns;
    const size_t single = (size_t)((p.M + 31) / 32) * ((p.N + 31) / 32) * zdim;
    pl.nb = (p.N > 32 && single > (size_t)3 * st.num_cu) ? 2 : 1;
    pl.lds = (size_t)(1 + pl.nb) * PG_PANEL * sizeof(float);  // 52 KB or 78 KB
    pl.grid = dim3((p.M + 31) / 32, (p.N + 32 * pl.nb - 1) / (32 * pl.nb), (unsigned)zdim);
    if (pl.grid.y > 65535u || zdim > 65535u) {
        set_error("panel product: grid too large");
        return 1;
    }
    return 0;
}

static int launch_panel_reduce(PanelArgs &p) {
    if (p.groups <= 1) return 0;
    hipLaunchKernelGGL(panel_reduce_kernel, dim3((unsigned)(((size_t)p.N * p.M + 255) / 256), p.nout), dim3(256), 0,
                       state().stream, p);
    p.groups = 0;  // (added up: a later call finds nothing to do)
    return hip_ok(hipGetLastError(), "panel reduce launch") ? 0 : 2;
}

// The additions of two products' sample groups in one launch.
static int launch_panel_reduce_pair(PanelArgs &p0, PanelArgs &p1) {
    if (p0.groups <= 1) return launch_panel_reduce(p1);
    if (p1.groups <= 1) return launch_panel_reduce(p0);
    const size_t nm0 = (size_t)p0.N * p0.M, nm1 = (size_t)p1.N * p1.M, nm = nm0 > nm1 ? nm0 : nm1;
    hipLaunchKernelGGL(panel_reduce_pair_kernel, dim3((unsigned)((nm + 255) / 256), p0.nout + p1.nout), dim3(256), 0,
                       state().stream, p0, p1);
    p0.groups = p1.groups = 0;
    return hip_ok(hipGetLastError(), "panel reduce launch") ? 0 : 2;
}

// Launches the panel product; `p` carries operands, strides and sizes, this fills in the rest.  In gradient
// mode (sum_samples) the partial sums of the sample groups go to `part` and a second kernel adds them.
static int launch_panel(PanelArgs &p, float *part) {
    State &st = state();
    PanelPlan pl;
    if (int rc = panel_plan(p, part, pl)) return rc;
    const bool ak = pl.ak, bk = pl.bk;
    void (*kern)(PanelArgs);
    if (pl.nb == 2)
        kern = ak ? (bk ? panel_gemm_kernel<true, true, 2> : panel_gemm_kernel<true, false, 2>)
                  : (bk ? panel_gemm_kernel<false, true, 2> : panel_gemm_kernel<false, false, 2>);
    else
        kern = ak ? (bk ? panel_gemm_kernel<true, true, 1> : panel_gemm_kernel<true, false, 1>)
                  : (bk ? panel_gemm_kernel<false, true, 1> : panel_gemm_kernel<false, false, 1>);
    if (pl.nb == 2) {
        static bool attr_set[4] = {false, false, false, false};
        const int which = (ak ? 2 : 0) + (bk ? 1 : 0);
        if (!attr_set[which]) {
            if (!hip_ok(hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)pl.lds),
                        "hipFuncSetAttribute"))
                return 2;
            attr_set[which] = true;
        }
    }
    hipLaunchKernelGGL(kern, pl.grid, dim3(ATT_NT * pl.nb), pl.lds, st.stream, p);
    if (!hip_ok(hipGetLastError(), "panel product launch")) return 2;
    return launch_panel_reduce(p);
}

// Two independent panel products in one launch (the two the backward pass has twice: the gradient of the output
// weights with the gradient of the attention map, and the gradients of the input weights with the gradient of the
// input), each followed by the addition of its sample groups where it has any.  `PAIR` names the orientations.
template <bool AK0, bool BK0, bool AK1, bool BK1>
static int launch_panel_pair(PanelArgs &p0, float *part0, PanelArgs &p1, float *part1, bool add_now = true) {
    State &st = state();
    PanelPlan l0, l1;
    if (int rc = panel_plan(p0, part0, l0)) return rc;
    if (int rc = panel_plan(p1, part1, l1)) return rc;
    const size_t n0 = (size_t)l0.grid.x * l0.grid.y * l0.grid.z, n1 = (size_t)l1.grid.x * l1.grid.y * l1.grid.z;
    if (l0.ak != AK0 || l0.bk != BK0 || l1.ak != AK1 || l1.bk != BK1 || n0 + n1 >= ((size_t)1 << 31) ||
        st.gemm_path == 7) {  // (not this pair, or one product at a time asked for)
        if (int rc = launch_panel(p0, part0)) return rc;
        return launch_panel(p1, part1);
    }
    void (*kern)(PanelArgs, PanelArgs, PanelPairGrid) = panel_gemm_pair_kernel<AK0, BK0, AK1, BK1>;
    const size_t lds = l0.lds > l1.lds ? l0.lds : l1.lds;
    static bool attr_set = false;
    if (!attr_set) {
        if (!hip_ok(hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                        (int)(3 * PG_PANEL * sizeof(float))),
                    "hipFuncSetAttribute"))
            return 2;
        attr_set = true;
    }
    PanelPairGrid g;
    g.n0 = (unsigned)n0;
    g.gx0 = l0.grid.x; g.gy0 = l0.grid.y;
    g.gx1 = l1.grid.x; g.gy1 = l1.grid.y;
    g.nb0 = l0.nb; g.nb1 = l1.nb;
    const int nbmax = l0.nb > l1.nb ? l0.nb : l1.nb;
    hipLaunchKernelGGL(kern, dim3((unsigned)(n0 + n1)), dim3(ATT_NT * nbmax), lds, st.stream, p0, p1, g);
    if (!hip_ok(hipGetLastError(), "panel product pair launch")) return 2;
    return add_now ? launch_panel_reduce_pair(p0, p1) : 0;  // (else the caller adds the groups up later)
}

// out[b][N x L] = Wt(N x K) . act[b][K x L]: a weight matrix with element (n,k) at n*a_n + k*a_k against a
// batch of activations (tokens contiguous).
static PanelArgs weights_times_acts(int N, int K, int L, int ns, int a_n, int a_k) {
    PanelArgs p = {};
    p.nout = p.nterm = 1;
    p.N = N;
    p.M = L;
    p.K = K;
    p.a_n = a_n;
    p.a_k = a_k;
    p.b_m = 1;
    p.b_k = L;
    p.b_s = (long long)K * L;
    p.c_s = (long long)N * L;
    p.c_n = L;
    p.ns = ns;
    return p;
}

// out[N x M] = sum over samples and tokens of A[b][N x L] . B[b][M x L]^T  (weight gradients).
static PanelArgs acts_times_acts(int N, int M, int L, int ns) {
    PanelArgs p = {};
    p.nout = p.nterm = 1;
    p.N = N;
    p.M = M;
    p.K = L;
    p.a_n = L;
    p.a_k = 1;
    p.a_s = (long long)N * L;
    p.b_m = L;
    p.b_k = 1;
    p.b_s = (long long)M * L;
    p.c_n = M;
    p.ns = ns;
    p.sum_samples = 1;
    return p;
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
    {
        // q/k/v[F x L] = W^T . X + bias in one launch (weights stored E x F: lib/sources/pulp_mhsa_fp32.c:70-325)
        PanelArgs p = weights_times_acts(F, E, L, ns, 1, F);
        p.nout = 3;
        for (int j = 0; j < 3; ++j) {
            p.A[j] = W[j];
            p.B[j] = X;
            p.C[j] = QKV[j];
            p.bias[j] = bias[j];
        }
        rc = launch_panel(p, nullptr);
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
    if (rc == 0) {
        // output[E x L] = Wout[E x F] . attention_map (:599-609)
        PanelArgs p = weights_times_acts(E, F, L, ns, F, 1);
        p.A[0] = Wo;
        p.B[0] = att;
        p.C[0] = Y;
        rc = launch_panel(p, nullptr);
    }
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
    const size_t p1 = panel_part_floats(1, E, F, ns), p3 = panel_part_floats(3, F, E, ns);
    float *rs = static_cast<float *>(scratch((rows + p1 + p3) * sizeof(float)));
    if (!rs) return 2;
    float *part_o = rs + rows, *part_i = part_o + p1;  // sample-group sums of the output / the input weights' gradients
    int rc = 0;
    // dWout[E x F] = sum over samples of dY . att^T (:742-760) and datt[F x L] = Wout^T . dY (:816-834), one launch;
    // the sample groups of dWout are added up at the end, together with those of the input weights' gradients
    PanelArgs pwo = acts_times_acts(E, F, L, ns);
    {
        pwo.A[0] = dY;
        pwo.B[0] = att;
        pwo.C[0] = dWo;
        PanelArgs q = weights_times_acts(F, E, L, ns, 1, F);
        q.A[0] = Wo;
        q.B[0] = dY;
        q.C[0] = datt;
        rc = launch_panel_pair<true, true, false, false>(pwo, part_o, q, nullptr, false);
    }
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
    if (rc == 0) {
        // dW_{q,k,v}[F x E] = sum over samples of d{q,k,v} . X^T (:1425-1560) and
        // dX[E x L] += W_q . dq + W_k . dk + W_v . dv (:1589-1745), one launch
        PanelArgs p = acts_times_acts(F, E, L, ns);
        p.nout = 3;
        for (int j = 0; j < 3; ++j) {
            p.A[j] = dQKV[j];
            p.B[j] = X;
            p.C[j] = dW[j];
        }
        PanelArgs q = weights_times_acts(E, F, L, ns, F, 1);
        q.nterm = 3;
        for (int j = 0; j < 3; ++j) {
            q.A[j] = W[j];
            q.B[j] = dQKV[j];
        }
        q.C[0] = dX;
        q.accumulate = 1;
        rc = launch_panel_pair<true, true, true, false>(p, part_i, q, nullptr, false);
        if (rc == 0) rc = launch_panel_reduce_pair(pwo, p);
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
