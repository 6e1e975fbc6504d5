// MFMA GEMM over separable index maps: C(n,m) = sum_k A(n,k) * B(m,k).
//
// One kernel family serves every GEMM-shaped step of the training core.  The
// two operands are described by separable index maps (ptl_common.hpp), so the
// implicit im2col gathers of Conv2D forward / weight-gradient / input-gradient,
// the batched pointwise and Linear products and the plain mm() contract are
// all the same code: only the maps differ.  Patch matrices are never
// materialised; patch elements are gathered from the tensor into the LDS tile.
//
// Work decomposition (gfx950, 64-wide waves):
//   * workgroup = 256 threads = 4 waves, computes a BM x BN tile of C;
//   * k is consumed in slabs of 64 bytes per row (32 halves or 16 floats),
//     staged global -> registers -> LDS with two LDS buffers, one barrier per
//     slab; LDS rows are k-contiguous with an 80-byte pitch so every MFMA
//     operand fragment is one 16-byte LDS read;
//   * fp16: v_mfma_f32_32x32x16_f16 (fp32 accumulate); fp32: v_mfma_f32_32x32x2_f32;
//   * optional split-K: grid.y slices k, fp32 partials go to a workspace and a
//     second kernel sums them in a fixed order (deterministic).
#include "ptl_common.hpp"

namespace ptl {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));

template <typename T>
struct Traits;
template <>
struct Traits<float> {
    static constexpr int VEC = 4;   // elements per 16-byte vector
    static constexpr int BKE = 16;  // elements of k per slab
};
template <>
struct Traits<half_t> {
    static constexpr int VEC = 8;
    static constexpr int BKE = 32;
};

constexpr int PITCH = 80;      // bytes per LDS tile row: 64 data + 16 pad
constexpr int KW = 512;        // k indices decoded per look-up window
constexpr int HW_BIAS = 8192;  // coordinate bias of packed look-up entries

// Look-up entry of one row or k index: x = element offset, y = packed
// (h + bias) << 16 | (w + bias).  An index outside [lo, hi) gets h-field 0,
// which fails the box test against any partner.
__device__ inline int2 lut_entry(const AxisMap &a, int idx, int lo, int hi) {
    int2 e;
    if (idx >= lo && idx < hi) {
        int off, h, w;
        axis_decode(a, idx, off, h, w);
        e.x = off;
        e.y = ((h + HW_BIAS) << 16) | (w + HW_BIAS);
    } else {
        e.x = 0;
        e.y = HW_BIAS;
    }
    return e;
}

__device__ inline bool box_ok(int2 rp, int2 kp, int HL, int WL) {
    unsigned s = (unsigned)rp.y + (unsigned)kp.y;
    int h = (int)(s >> 16) - 2 * HW_BIAS;
    int w = (int)(s & 0xffffu) - 2 * HW_BIAS;
    return ((unsigned)h < (unsigned)HL) && ((unsigned)w < (unsigned)WL);
}

template <typename T>
union Stage {
    uint4 v[4];
    T e[64 / sizeof(T)];
};

// Fetch this thread's share of an R-row operand slab into registers.
// kl = slab start relative to the look-up window, kg = absolute slab start.
template <typename T, int R>
__device__ inline void load_stage(Stage<T> &st, const T *__restrict__ base, const OperandMap &om,
                                  const int2 *rlut, const int2 *klut, int kl, int kg, int kend,
                                  int tid) {
    constexpr int VEC = Traits<T>::VEC, BKE = Traits<T>::BKE;
    const int mode = om.mode;
    if (mode == FILL_VEC_K) {
        constexpr int NCH = (R * 4 + 255) / 256;
#pragma unroll
        for (int i = 0; i < NCH; ++i) {
            int c = tid + i * 256;
            uint4 v = make_uint4(0, 0, 0, 0);
            if (c < R * 4) {
                int row = c >> 2, kc = c & 3;
                int2 rp = rlut[row];
                int2 kp = klut[kl + kc * VEC];
                if ((rp.y >> 16) != 0 && (kp.y >> 16) != 0)
                    v = *reinterpret_cast<const uint4 *>(base + rp.x + kp.x);
            }
            st.v[i] = v;
        }
    } else if (mode == FILL_VEC_R) {
        constexpr int RV = R / VEC;  // row vectors per k
        if (tid < R) {
            int rv = tid % RV, kq = tid / RV;
            int2 rp = rlut[rv * VEC];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                int2 kp = klut[kl + kq * 4 + i];
                uint4 v = make_uint4(0, 0, 0, 0);
                if ((rp.y >> 16) != 0 && (kp.y >> 16) != 0)
                    v = *reinterpret_cast<const uint4 *>(base + rp.x + kp.x);
                st.v[i] = v;
            }
        }
    } else if (mode == FILL_ELEM_R) {
        constexpr int SLOTS = 256 / R, PER = BKE / SLOTS;
        int row = tid % R, slot = tid / R;
        int2 rp = rlut[row];
#pragma unroll
        for (int j = 0; j < PER; ++j) {
            int2 kp = klut[kl + slot + j * SLOTS];
            T x = (T)0;
            if (box_ok(rp, kp, om.HL, om.WL)) x = base[rp.x + kp.x];
            st.e[j] = x;
        }
    } else {  // FILL_ELEM_K
        constexpr int RSLOTS = 256 / BKE, PER = R / RSLOTS;
        int kk = tid % BKE, rs = tid / BKE;
        int2 kp = klut[kl + kk];
#pragma unroll
        for (int j = 0; j < PER; ++j) {
            int2 rp = rlut[rs + j * RSLOTS];
            T x = (T)0;
            if (box_ok(rp, kp, om.HL, om.WL)) x = base[rp.x + kp.x];
            st.e[j] = x;
        }
    }
}

// Write the staged registers into an LDS tile (rows k-contiguous, PITCH bytes).
template <typename T, int R>
__device__ inline void store_stage(const Stage<T> &st, char *tile, int mode, int tid) {
    constexpr int VEC = Traits<T>::VEC, BKE = Traits<T>::BKE;
    if (mode == FILL_VEC_K) {
        constexpr int NCH = (R * 4 + 255) / 256;
#pragma unroll
        for (int i = 0; i < NCH; ++i) {
            int c = tid + i * 256;
            if (c < R * 4) {
                int row = c >> 2, kc = c & 3;
                *reinterpret_cast<uint4 *>(tile + row * PITCH + kc * 16) = st.v[i];
            }
        }
    } else if (mode == FILL_VEC_R) {
        constexpr int RV = R / VEC;
        if (tid < R) {
            int rv = tid % RV, kq = tid / RV;
            // st.v[i] holds VEC consecutive rows at k = kq*4 + i: transpose to
            // one 4-wide k run per row.
#pragma unroll
            for (int j = 0; j < VEC; ++j) {
                alignas(16) T q[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) q[i] = st.e[i * VEC + j];
                char *p = tile + (rv * VEC + j) * PITCH + kq * 4 * (int)sizeof(T);
                if (sizeof(T) == 4) {
                    *reinterpret_cast<uint4 *>(p) = *reinterpret_cast<const uint4 *>(q);
                } else {
                    *reinterpret_cast<uint2 *>(p) = *reinterpret_cast<const uint2 *>(q);
                }
            }
        }
    } else if (mode == FILL_ELEM_R) {
        constexpr int SLOTS = 256 / R, PER = BKE / SLOTS;
        int row = tid % R, slot = tid / R;
#pragma unroll
        for (int j = 0; j < PER; ++j)
            *reinterpret_cast<T *>(tile + row * PITCH + (slot + j * SLOTS) * (int)sizeof(T)) = st.e[j];
    } else {
        constexpr int RSLOTS = 256 / BKE, PER = R / RSLOTS;
        int kk = tid % BKE, rs = tid / BKE;
#pragma unroll
        for (int j = 0; j < PER; ++j)
            *reinterpret_cast<T *>(tile + (rs + j * RSLOTS) * PITCH + kk * (int)sizeof(T)) = st.e[j];
    }
}

template <typename T>
__device__ inline void mfma_slab(f32x16 &acc, const uint4 &a, const uint4 &b);

template <>
__device__ inline void mfma_slab<half_t>(f32x16 &acc, const uint4 &a, const uint4 &b) {
    f16x8 av = __builtin_bit_cast(f16x8, a);
    f16x8 bv = __builtin_bit_cast(f16x8, b);
    acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(av, bv, acc, 0, 0, 0);
}

template <>
__device__ inline void mfma_slab<float>(f32x16 &acc, const uint4 &a, const uint4 &b) {
    f32x4 av = __builtin_bit_cast(f32x4, a);
    f32x4 bv = __builtin_bit_cast(f32x4, b);
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(av.x, bv.x, acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(av.y, bv.y, acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(av.z, bv.z, acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(av.w, bv.w, acc, 0, 0, 0);
}

template <typename T, int BM, int BN, int WAVES_M, int WAVES_N>
__global__ __launch_bounds__(256) void gemm_kernel(const GemmArgs g) {
    constexpr int BKE = Traits<T>::BKE;
    constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
    constexpr int FM = WM / 32, FN = WN / 32;
    static_assert(WAVES_M * WAVES_N == 4, "four waves per workgroup");
    static_assert(FM >= 1 && FN >= 1, "wave tile is a multiple of 32x32");

    __shared__ __attribute__((aligned(16))) char tileA[2][BM * PITCH];
    __shared__ __attribute__((aligned(16))) char tileB[2][BN * PITCH];
    __shared__ int2 rlutA[BM];
    __shared__ int2 rlutB[BN];
    __shared__ int2 klutA[KW];
    __shared__ int2 klutB[KW];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;

    const int tile = blockIdx.x;
    const int z = blockIdx.y;
    const int tn = tile / g.tiles_m, tm = tile % g.tiles_m;
    const int n0 = tn * BM, m0 = tm * BN;
    const int kbeg = z * g.kchunk;
    const int kend = min(g.K, kbeg + g.kchunk);

    const T *__restrict__ Ab = reinterpret_cast<const T *>(g.A);
    const T *__restrict__ Bb = reinterpret_cast<const T *>(g.B);

    for (int i = tid; i < BM; i += 256) rlutA[i] = lut_entry(g.a.row, n0 + i, 0, g.N);
    for (int i = tid; i < BN; i += 256) rlutB[i] = lut_entry(g.b.row, m0 + i, 0, g.M);

    f32x16 acc[FM][FN];
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

    const int a_mode = g.a.mode, b_mode = g.b.mode;
    const int frag_off = (lane & 31) * PITCH + (lane >> 5) * 16;

    for (int kw = kbeg; kw < kend; kw += KW) {
        const int kwe = min(kw + KW, kend);
        __syncthreads();
        for (int i = tid; i < KW; i += 256) {
            klutA[i] = lut_entry(g.a.k, kw + i, kw, kwe);
            klutB[i] = lut_entry(g.b.k, kw + i, kw, kwe);
        }
        __syncthreads();
        const int nsteps = (kwe - kw + BKE - 1) / BKE;

        Stage<T> sa, sb;
        load_stage<T, BM>(sa, Ab, g.a, rlutA, klutA, 0, kw, kwe, tid);
        load_stage<T, BN>(sb, Bb, g.b, rlutB, klutB, 0, kw, kwe, tid);
        store_stage<T, BM>(sa, tileA[0], a_mode, tid);
        store_stage<T, BN>(sb, tileB[0], b_mode, tid);
        __syncthreads();

        for (int s = 0; s < nsteps; ++s) {
            const bool more = (s + 1 < nsteps);
            if (more) {
                load_stage<T, BM>(sa, Ab, g.a, rlutA, klutA, (s + 1) * BKE, kw + (s + 1) * BKE, kwe, tid);
                load_stage<T, BN>(sb, Bb, g.b, rlutB, klutB, (s + 1) * BKE, kw + (s + 1) * BKE, kwe, tid);
            }
            const char *pa = tileA[s & 1] + wm * WM * PITCH + frag_off;
            const char *pb = tileB[s & 1] + wn * WN * PITCH + frag_off;
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                uint4 af[FM], bf[FN];
#pragma unroll
                for (int i = 0; i < FM; ++i)
                    af[i] = *reinterpret_cast<const uint4 *>(pa + i * 32 * PITCH + h * 32);
#pragma unroll
                for (int j = 0; j < FN; ++j)
                    bf[j] = *reinterpret_cast<const uint4 *>(pb + j * 32 * PITCH + h * 32);
#pragma unroll
                for (int i = 0; i < FM; ++i)
#pragma unroll
                    for (int j = 0; j < FN; ++j) mfma_slab<T>(acc[i][j], af[i], bf[j]);
            }
            if (more) {
                store_stage<T, BM>(sa, tileA[(s + 1) & 1], a_mode, tid);
                store_stage<T, BN>(sb, tileB[(s + 1) & 1], b_mode, tid);
            }
            __syncthreads();
        }
    }

    // Epilogue.  Accumulator element v of fragment (i, j) in lane l is
    // C[row 8*(v/4) + 4*(l/32) + v%4][col l%32] of that 32x32 block.
    __syncthreads();
    int *nlut = reinterpret_cast<int *>(klutA);
    int *mlut = reinterpret_cast<int *>(klutB);
    if (g.splits == 1) {
        for (int i = tid; i < BM; i += 256) {
            int off = 0, h, w;
            if (n0 + i < g.N) axis_decode(g.c.n, n0 + i, off, h, w);
            nlut[i] = off;
        }
        for (int i = tid; i < BN; i += 256) {
            int off = 0, h, w;
            if (m0 + i < g.M) axis_decode(g.c.m, m0 + i, off, h, w);
            mlut[i] = off;
        }
        __syncthreads();
        T *__restrict__ Cb = reinterpret_cast<T *>(g.C);
#pragma unroll
        for (int i = 0; i < FM; ++i)
#pragma unroll
            for (int j = 0; j < FN; ++j) {
                int ml = wn * WN + j * 32 + (lane & 31);
                if (m0 + ml < g.M) {
                    int mo = mlut[ml];
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        int nl = wm * WM + i * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
                        if (n0 + nl < g.N) Cb[nlut[nl] + mo] = (T)acc[i][j][v];
                    }
                }
            }
    } else {
        float *__restrict__ ws = g.ws + (size_t)z * g.N * g.M;
#pragma unroll
        for (int i = 0; i < FM; ++i)
#pragma unroll
            for (int j = 0; j < FN; ++j) {
                int m = m0 + wn * WN + j * 32 + (lane & 31);
                if (m < g.M) {
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        int n = n0 + wm * WM + i * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
                        if (n < g.N) ws[(size_t)n * g.M + m] = acc[i][j][v];
                    }
                }
            }
    }
}

// Sum split-K partials (fixed order) and scatter through the output map: 64 outputs per
// workgroup, four split groups in parallel, four loads in flight per thread -- with few outputs
// and many splits the kernel lives on memory-level parallelism.
template <typename T>
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float *__restrict__ ws, T *__restrict__ C,
                                                            OutMap c, int N, int M, int splits) {
    __shared__ float part[4][64];
    const size_t total = (size_t)N * M;
    const int o = threadIdx.x & 63, sg = threadIdx.x >> 6;
    const size_t idx = (size_t)blockIdx.x * 64 + o;
    float s = 0.f;
    if (idx < total) {
        const float *src = ws + idx;
        int z = sg;
        for (; z + 3 * 4 < splits; z += 4 * 4) {
            float v[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) v[u] = src[(size_t)(z + u * 4) * total];
#pragma unroll
            for (int u = 0; u < 4; ++u) s += v[u];
        }
        for (; z < splits; z += 4) s += src[(size_t)z * total];
    }
    part[sg][o] = s;
    __syncthreads();
    if (sg != 0 || idx >= total) return;
    s += part[1][o] + part[2][o] + part[3][o];
    int n = (int)(idx / M), m = (int)(idx % M);
    int on, om, h, w;
    axis_decode(c.n, n, on, h, w);
    axis_decode(c.m, m, om, h, w);
    C[on + om] = (T)s;
}

// ---------------------------------------------------------------------------
// Host side: operand fill mode, tile shape and split selection, launch.
// ---------------------------------------------------------------------------
static bool axis_is_single(const AxisMap &a) { return a.d0 >= a.n; }

static bool no_coords(const AxisMap &a) {
    return a.h2 == 0 && a.h1 == 0 && a.h0 == 0 && a.hb == 0 && a.w2 == 0 && a.w1 == 0 && a.w0 == 0 &&
           a.wb == 0;
}

static bool mult(const AxisMap &a, int v, bool include_o0) {
    return a.o2 % v == 0 && a.o1 % v == 0 && a.ob % v == 0 && (!include_o0 || a.o0 % v == 0);
}

template <typename T>
static int choose_mode(const OperandMap &om, const void *base, int rows, int K) {
    constexpr int VEC = Traits<T>::VEC;
    bool plain_box = no_coords(om.row) && no_coords(om.k) && om.HL >= 1 && om.WL >= 1;
    bool aligned = (reinterpret_cast<uintptr_t>(base) % 16) == 0;
    if (plain_box && aligned) {
        // contiguous along k: a 16-byte vector must stay inside one q0 run
        if (om.k.o0 == 1 && (axis_is_single(om.k) || om.k.d0 % VEC == 0) && K % VEC == 0 &&
            mult(om.k, VEC, false) && mult(om.row, VEC, true))
            return FILL_VEC_K;
        if (om.row.o0 == 1 && (axis_is_single(om.row) || om.row.d0 % VEC == 0) && rows % VEC == 0 &&
            mult(om.row, VEC, false) && mult(om.k, VEC, true))
            return FILL_VEC_R;
    }
    // Element gather: consecutive lanes walk the axis whose unit-stride runs are longer (for an
    // implicit im2col that is the pixel axis: a row of the image against a row of the filter).
    auto run = [](const AxisMap &a) {
        int s = a.o0 < 0 ? -a.o0 : a.o0;
        int len = a.d0 < a.n ? a.d0 : a.n;
        return s == 1 ? len : 0;
    };
    int rk = run(om.k), rr = run(om.row);
    if (rk != rr) return rk > rr ? FILL_ELEM_K : FILL_ELEM_R;
    int ak = om.k.o0 < 0 ? -om.k.o0 : om.k.o0;
    int ar = om.row.o0 < 0 ? -om.row.o0 : om.row.o0;
    return ak <= ar ? FILL_ELEM_K : FILL_ELEM_R;
}

template <typename T, int BM, int BN, int WMv, int WNv>
static void launch_cfg(GemmArgs &g, hipStream_t s) {
    g.tiles_n = (g.N + BM - 1) / BM;
    g.tiles_m = (g.M + BN - 1) / BN;
    dim3 grid(g.tiles_n * g.tiles_m, g.splits);
    hipLaunchKernelGGL((gemm_kernel<T, BM, BN, WMv, WNv>), grid, dim3(256), 0, s, g);
}

// Tile shape, split selection and launch of the staged kernel.
template <typename T>
static int launch_staged(GemmArgs &g) {
    State &st = state();
    constexpr int BKE = Traits<T>::BKE;
    // Tile shape: skinny outputs get a 32-row (or 32-column) tile; otherwise the
    // largest square tile that still yields at least one workgroup per CU.
    int cfg;
    auto tiles = [&](int bm, int bn) { return (long)((g.N + bm - 1) / bm) * ((g.M + bn - 1) / bn); };
    if (g.N <= 32)
        cfg = 2;
    else if (g.M <= 32)
        cfg = 3;
    else if (tiles(128, 128) >= st.num_cu)
        cfg = 0;
    else
        cfg = 1;
    long nt = cfg == 0 ? tiles(128, 128) : cfg == 1 ? tiles(64, 64) : cfg == 2 ? tiles(32, 128) : tiles(128, 32);

    // Split k when the output alone cannot fill the machine.
    g.splits = 1;
    g.kchunk = ((g.K + BKE - 1) / BKE) * BKE;
    if (nt * 2 <= st.num_cu) {
        int min_chunk = 4 * BKE;
        int max_splits = (g.K + min_chunk - 1) / min_chunk;
        int want = (int)((st.num_cu + nt - 1) / nt);
        int sp = want < max_splits ? want : max_splits;
        if (sp > 1) {
            int chunk = (g.K + sp - 1) / sp;
            chunk = ((chunk + BKE - 1) / BKE) * BKE;
            sp = (g.K + chunk - 1) / chunk;
            if (sp > 1) {
                g.splits = sp;
                g.kchunk = chunk;
            }
        }
    }
    if (g.splits > 1) {
        g.ws = workspace((size_t)g.splits * g.N * g.M * sizeof(float));
        if (!g.ws) return 2;
    }
    switch (cfg) {
        case 0: launch_cfg<T, 128, 128, 2, 2>(g, st.stream); break;
        case 1: launch_cfg<T, 64, 64, 2, 2>(g, st.stream); break;
        case 2: launch_cfg<T, 32, 128, 1, 4>(g, st.stream); break;
        default: launch_cfg<T, 128, 32, 4, 1>(g, st.stream); break;
    }
    return hip_ok(hipGetLastError(), "gemm launch") ? 0 : 2;
}

template <typename T>
int gemm(const GemmArgs &gin) {
    if (!ensure_init()) return 2;
    GemmArgs g = gin;
    if (g.N <= 0 || g.M <= 0 || g.K <= 0) return 0;
    State &st = state();

    g.a.mode = choose_mode<T>(g.a, g.A, g.N, g.K);
    g.b.mode = choose_mode<T>(g.b, g.B, g.M, g.K);

    int rc = -1;
    if (st.gemm_path != 1) rc = gemm_async<T>(g);
    if (rc > 0) return rc;
    if (rc < 0) {
        rc = launch_staged<T>(g);
        if (rc) return rc;
    }
    if (g.splits > 1) {
        size_t total = (size_t)g.N * g.M;
        hipLaunchKernelGGL((splitk_reduce_kernel<T>), dim3((unsigned)((total + 63) / 64)), dim3(256), 0,
                           st.stream, g.ws, reinterpret_cast<T *>(g.C), g.c, g.N, g.M, g.splits);
        if (!hip_ok(hipGetLastError(), "split-k reduce launch")) return 2;
    }
    return 0;
}

template <typename T>
int gemm_pair(const GemmArgs &g0in, const GemmArgs &g1in) {
    if (!ensure_init()) return 2;
    GemmArgs g0 = g0in, g1 = g1in;
    if (state().gemm_path == 0 && g0.N > 0 && g0.M > 0 && g0.K > 0 && g1.N > 0 && g1.M > 0 && g1.K > 0) {
        g0.a.mode = choose_mode<T>(g0.a, g0.A, g0.N, g0.K);
        g0.b.mode = choose_mode<T>(g0.b, g0.B, g0.M, g0.K);
        g1.a.mode = choose_mode<T>(g1.a, g1.A, g1.N, g1.K);
        g1.b.mode = choose_mode<T>(g1.b, g1.B, g1.M, g1.K);
        int rc = gemm_async_pair<T>(g0, g1);
        if (rc >= 0) return rc;
    }
    int rc = gemm<T>(g0in);
    return rc ? rc : gemm<T>(g1in);
}

template int gemm_pair<float>(const GemmArgs &, const GemmArgs &);
template int gemm_pair<half_t>(const GemmArgs &, const GemmArgs &);
template int gemm<float>(const GemmArgs &);
template int gemm<half_t>(const GemmArgs &);

// ---------------------------------------------------------------------------
// Products with a unit dimension (Linear at batch 1): bandwidth-bound kernels.
// ---------------------------------------------------------------------------

// y[r] = sum_k Mx[r*K + k] * x[k]; one wave per row.
template <typename T>
__global__ __launch_bounds__(256) void gemv_rowdot_kernel(const T *__restrict__ Mx, const T *__restrict__ x,
                                                          T *__restrict__ y, int R, int K, int vec_ok) {
    constexpr int VEC = Traits<T>::VEC;
    int row = blockIdx.x * 4 + (threadIdx.x >> 6);
    int lane = threadIdx.x & 63;
    if (row >= R) return;
    const T *p = Mx + (size_t)row * K;
    float s = 0.f;
    if (vec_ok) {
        for (int k = lane * VEC; k < K; k += 64 * VEC) {
            Stage<T> a, b;
            a.v[0] = *reinterpret_cast<const uint4 *>(p + k);
            b.v[0] = *reinterpret_cast<const uint4 *>(x + k);
#pragma unroll
            for (int i = 0; i < VEC; ++i) s += (float)a.e[i] * (float)b.e[i];
        }
    } else {
        for (int k = lane; k < K; k += 64) s += (float)p[k] * (float)x[k];
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) s += __shfl_down(s, o, 64);
    if (lane == 0) y[row] = (T)s;
}

// part[z][m] = sum_{k in slice z} x[k] * Mx[k*M + m]
template <typename T>
__global__ __launch_bounds__(256) void gemv_coldot_kernel(const T *__restrict__ x, const T *__restrict__ Mx,
                                                          float *__restrict__ part, int K, int M, int kchunk) {
    int m = blockIdx.x * 256 + threadIdx.x;
    if (m >= M) return;
    int k0 = blockIdx.y * kchunk;
    int k1 = min(K, k0 + kchunk);
    float s = 0.f;
    for (int k = k0; k < k1; ++k) s += (float)x[k] * (float)Mx[(size_t)k * M + m];
    part[(size_t)blockIdx.y * M + m] = s;
}

// Same product with 16-byte loads: a workgroup owns CV*VEC consecutive columns and a
// slice of k; thread (kl, cv) sums rows k0+kl, k0+kl+32, ... of column vector cv, the
// 32 row-lanes are then folded through LDS.
template <typename T>
__global__ __launch_bounds__(256) void gemv_coldot_vec_kernel(const T *__restrict__ x, const T *__restrict__ Mx,
                                                              float *__restrict__ part, int K, int M, int kchunk) {
    constexpr int VEC = Traits<T>::VEC, CV = 8, KL = 256 / CV;
    const int cv = threadIdx.x % CV, kl = threadIdx.x / CV;
    const int col = (blockIdx.x * CV + cv) * VEC;
    const int k0 = blockIdx.y * kchunk, k1 = min(K, k0 + kchunk);
    float acc[VEC];
#pragma unroll
    for (int i = 0; i < VEC; ++i) acc[i] = 0.f;
    if (col < M) {
        for (int k = k0 + kl; k < k1; k += KL) {
            Stage<T> v;
            v.v[0] = *reinterpret_cast<const uint4 *>(Mx + (size_t)k * M + col);
            float xv = (float)x[k];
#pragma unroll
            for (int i = 0; i < VEC; ++i) acc[i] += xv * (float)v.e[i];
        }
    }
    __shared__ float red[KL][CV * VEC + 1];
#pragma unroll
    for (int i = 0; i < VEC; ++i) red[kl][cv * VEC + i] = acc[i];
    __syncthreads();
    if (threadIdx.x < CV * VEC) {
        float s = 0.f;
#pragma unroll 8
        for (int r = 0; r < KL; ++r) s += red[r][threadIdx.x];
        int c = blockIdx.x * CV * VEC + threadIdx.x;
        if (c < M) part[(size_t)blockIdx.y * M + c] = s;
    }
}

// The same product in ONE launch for moderate K: a workgroup owns 4*VEC consecutive columns and
// ALL rows; thread (kl, cv) sums rows kl, kl+64, ... of column vector cv with eight loads in
// flight, the 64 row-lanes are folded through LDS.  (A cross-workgroup "last arriver adds the
// partials" variant was tried: the device-scope fences it needs write back the whole L2 per
// workgroup and made it twice as slow as two launches.)
template <typename T>
__global__ __launch_bounds__(256) void gemv_coldot_whole_kernel(const T *__restrict__ x, const T *__restrict__ Mx,
                                                                T *__restrict__ y, int K, int M) {
    constexpr int VEC = Traits<T>::VEC, CV = 4, KL = 256 / CV;
    const int cv = threadIdx.x % CV, kl = threadIdx.x / CV;
    const int col = (blockIdx.x * CV + cv) * VEC;
    float acc[VEC];
#pragma unroll
    for (int i = 0; i < VEC; ++i) acc[i] = 0.f;
    if (col < M) {
        const T *p = Mx + col;
        int k = kl;
        for (; k + 7 * KL < K; k += 8 * KL) {
            Stage<T> v[8];
            float xv[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                v[u].v[0] = *reinterpret_cast<const uint4 *>(p + (size_t)(k + u * KL) * M);
                xv[u] = (float)x[k + u * KL];
            }
#pragma unroll
            for (int u = 0; u < 8; ++u)
#pragma unroll
                for (int i = 0; i < VEC; ++i) acc[i] += xv[u] * (float)v[u].e[i];
        }
        for (; k < K; k += KL) {
            Stage<T> v;
            v.v[0] = *reinterpret_cast<const uint4 *>(p + (size_t)k * M);
            const float xv = (float)x[k];
#pragma unroll
            for (int i = 0; i < VEC; ++i) acc[i] += xv * (float)v.e[i];
        }
    }
    __shared__ float red[KL][CV * VEC + 1];
#pragma unroll
    for (int i = 0; i < VEC; ++i) red[kl][cv * VEC + i] = acc[i];
    __syncthreads();
    if (threadIdx.x < CV * VEC) {
        float s = 0.f;
#pragma unroll 8
        for (int r = 0; r < KL; ++r) s += red[r][threadIdx.x];
        const int c = blockIdx.x * CV * VEC + threadIdx.x;
        if (c < M) y[c] = (T)s;
    }
}

template <typename T>
__global__ __launch_bounds__(256) void colsum_reduce_kernel(const float *__restrict__ part, T *__restrict__ y,
                                                            int M, int splits) {
    int m = blockIdx.x * 256 + threadIdx.x;
    if (m >= M) return;
    float s = 0.f;
    for (int z = 0; z < splits; ++z) s += part[(size_t)z * M + m];
    y[m] = (T)s;
}

// C[n*M + m] = a[n] * b[m]
template <typename T>
__global__ __launch_bounds__(256) void outer_kernel(const T *__restrict__ a, const T *__restrict__ b,
                                                    T *__restrict__ C, int N, int M) {
    size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    size_t total = (size_t)N * M;
    if (idx >= total) return;
    int n = (int)(idx / M), m = (int)(idx % M);
    C[idx] = (T)((float)a[n] * (float)b[m]);
}

// Same with 16-byte stores (M a multiple of the vector, b and C 16-byte aligned): a thread owns VEC
// consecutive columns of four consecutive rows.
template <typename T>
__global__ __launch_bounds__(256) void outer_vec_kernel(const T *__restrict__ a, const T *__restrict__ b,
                                                        T *__restrict__ C, int N, int M) {
    constexpr int VEC = Traits<T>::VEC;
    const int mv = M / VEC;
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    const size_t total = (size_t)((N + 3) / 4) * mv;
    if (idx >= total) return;
    const int n0 = (int)(idx / mv) * 4, m = (int)(idx % mv) * VEC;
    Stage<T> bv, out;
    bv.v[0] = *reinterpret_cast<const uint4 *>(b + m);
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        if (n0 + r >= N) break;
        const float av = (float)a[n0 + r];
#pragma unroll
        for (int i = 0; i < VEC; ++i) out.e[i] = (T)(av * (float)bv.e[i]);
        *reinterpret_cast<uint4 *>(C + (size_t)(n0 + r) * M + m) = out.v[0];
    }
}

template <typename T>
static int gemv_rowdot(const T *Mx, const T *x, T *y, int R, int K) {
    constexpr int VEC = Traits<T>::VEC;
    State &st = state();
    int vec_ok = (K % VEC == 0) && (reinterpret_cast<uintptr_t>(Mx) % 16 == 0) &&
                 (reinterpret_cast<uintptr_t>(x) % 16 == 0);
    hipLaunchKernelGGL((gemv_rowdot_kernel<T>), dim3((R + 3) / 4), dim3(256), 0, st.stream, Mx, x, y, R, K,
                       vec_ok);
    return hip_ok(hipGetLastError(), "gemv launch") ? 0 : 2;
}

template <typename T>
int mm_dispatch(const T *A, const T *B, T *C, int N, int M, int K, int trans_B) {
    if (!ensure_init()) return 2;
    if (N <= 0 || M <= 0 || K <= 0) return 0;  // K == 0 leaves C untouched, as mm() does
    State &st = state();
    if (K == 1) {
        size_t total = (size_t)N * M;
        constexpr int VO = Traits<T>::VEC;
        if (M % VO == 0 && reinterpret_cast<uintptr_t>(B) % 16 == 0 && reinterpret_cast<uintptr_t>(C) % 16 == 0) {
            size_t units = (size_t)((N + 3) / 4) * (M / VO);
            hipLaunchKernelGGL((outer_vec_kernel<T>), dim3((unsigned)((units + 255) / 256)), dim3(256), 0, st.stream,
                               A, B, C, N, M);
            return hip_ok(hipGetLastError(), "outer launch") ? 0 : 2;
        }
        hipLaunchKernelGGL((outer_kernel<T>), dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st.stream, A,
                           B, C, N, M);
        return hip_ok(hipGetLastError(), "outer launch") ? 0 : 2;
    }
    if (M == 1) return gemv_rowdot<T>(A, B, C, N, K);  // B is K x 1 or 1 x K: the same vector
    if (N == 1 && trans_B) return gemv_rowdot<T>(B, A, C, M, K);
    constexpr int VECW = Traits<T>::VEC;
    if (N == 1 && M % VECW == 0 && reinterpret_cast<uintptr_t>(B) % 16 == 0) {
        const int colblk = 8 * VECW;
        int blocks_m = (M + colblk - 1) / colblk;
        int splits = (2 * st.num_cu + blocks_m - 1) / blocks_m;
        if (splits > (K + 31) / 32) splits = (K + 31) / 32;
        if (splits < 1) splits = 1;
        int kchunk = (K + splits - 1) / splits;
        splits = (K + kchunk - 1) / kchunk;
        float *part = workspace((size_t)splits * M * sizeof(float));
        if (!part) return 2;
        if (K <= 4096) {  // one launch: each workgroup sums whole columns
            hipLaunchKernelGGL((gemv_coldot_whole_kernel<T>), dim3((M + 4 * VECW - 1) / (4 * VECW)), dim3(256), 0,
                               st.stream, A, B, C, K, M);
            return hip_ok(hipGetLastError(), "gemv launch") ? 0 : 2;
        }
        hipLaunchKernelGGL((gemv_coldot_vec_kernel<T>), dim3(blocks_m, splits), dim3(256), 0, st.stream, A, B, part,
                           K, M, kchunk);
        hipLaunchKernelGGL((colsum_reduce_kernel<T>), dim3((M + 255) / 256), dim3(256), 0, st.stream, part, C, M,
                           splits);
        return hip_ok(hipGetLastError(), "gemv launch") ? 0 : 2;
    }
    if (N == 1) {
        int splits = (st.num_cu * 256 + M - 1) / M;  // about one thread-column per lane of the chip
        if (splits > K / 8) splits = K / 8;
        if (splits < 1) splits = 1;
        int kchunk = (K + splits - 1) / splits;
        splits = (K + kchunk - 1) / kchunk;
        float *part = workspace((size_t)splits * M * sizeof(float));
        if (!part) return 2;
        hipLaunchKernelGGL((gemv_coldot_kernel<T>), dim3((M + 255) / 256, splits), dim3(256), 0, st.stream, A,
                           B, part, K, M, kchunk);
        hipLaunchKernelGGL((colsum_reduce_kernel<T>), dim3((M + 255) / 256), dim3(256), 0, st.stream, part, C, M,
                           splits);
        return hip_ok(hipGetLastError(), "gemv launch") ? 0 : 2;
    }
    GemmArgs g = {};
    g.A = A;
    g.B = B;
    g.C = C;
    g.N = N;
    g.M = M;
    g.K = K;
    g.a.row = axis_plain(N, K);
    g.a.k = axis_plain(K, 1);
    g.a.HL = g.a.WL = 1;
    if (trans_B) {
        g.b.row = axis_plain(M, K);
        g.b.k = axis_plain(K, 1);
    } else {
        g.b.row = axis_plain(M, 1);
        g.b.k = axis_plain(K, M);
    }
    g.b.HL = g.b.WL = 1;
    g.c.n = axis_plain(N, M);
    g.c.m = axis_plain(M, 1);
    return gemm<T>(g);
}

template int mm_dispatch<float>(const float *, const float *, float *, int, int, int, int);
template int mm_dispatch<half_t>(const half_t *, const half_t *, half_t *, int, int, int, int);

}  // namespace ptl
