// Direct convolution on MFMA for channel-major (CHW) tensors: forward, and input
// gradient as a forward pass over the (zero-stuffed) output gradient with flipped,
// transposed filters.
//
// The GEMM route fetches every element of the implicit im2col matrix from global
// memory, Hk*Wk times per input element and one lane-load each.  Here a workgroup
// owns BM consecutive output pixels (raster order over sample, row, column) and BN
// output channels, and
//   * loads the input rows those pixels touch ONCE into LDS, as [channel block][row][col]
//     chunks of 16 bytes that hold VEC consecutive channels of one input position, the
//     padding halo written as zeros (raw tile).  A chunk is gathered with VEC strided
//     element loads, which a wave coalesces along the columns;
//   * loads its BN filters into LDS as [filter][tap][channel] (rows padded to an odd
//     multiple of 16 bytes, which spreads sixteen consecutive filters over all 64 banks),
//     once per workgroup: a workgroup then walks several pixel tiles;
//   * runs the contraction tap by tap, channel blocks innermost: the A fragment of a lane
//     (one pixel, VEC channels) is ONE ds_read_b128 at rawoff(pixel) + tapoff(hk, wk), the
//     B fragment another, i.e. the im2col matrix never exists, not even in LDS;
//   * parks the accumulators in LDS and stores whole lines along the pixel axis
//     (shared tile epilogue).
// Workgroups are small (BM/32 waves) and use little LDS, so several are resident per CU
// and hide each other's load, barrier and store phases.
#include "ptl_gemm_async.hpp"
#include "ptl_gemm_async.inc"
#include "ptl_conv_tile.hpp"
#include "ptl_host.hpp"

namespace ptl {

struct ConvTileArgs {
    const void *X;
    const void *Wt;
    GemmArgs g;  // epilogue view: C, c, N = pixels, M = filters, splits = 1
    ConvTileDesc d;
    int CinP;     // channels rounded up to the MFMA k step (extra planes are zero)
    int THP;      // rows of a padded input image
    int TW;       // columns of a padded input row
    int RR;       // raw rows a tile holds
    int PLANE;    // RR * TW
    int b_pitch;  // bytes per filter row in LDS
    int b_bytes;  // LDS bytes of the filter tile (the raw tile follows)
    int tiles;    // pixel tiles; a workgroup walks tiles blockIdx.x, blockIdx.x + gridDim.x, ...
    unsigned magic_tw, magic_rr, magic_perm, magic_cb, magic_kw;  // ceil(2^32 / d): exact for n, d < 2^16
    int c_mode;
};


template <typename T, int BM, int BN, int WAVES_K>
__global__ __launch_bounds__((BM / 32) * WAVES_K * 64) void conv_tile_kernel(const ConvTileArgs a) {
    constexpr int NT = (BM / 32) * WAVES_K * 64;
    constexpr int ES = (int)sizeof(T), VEC = 16 / ES, KSTEP = 2 * VEC, FN = BN / 32;
    extern __shared__ __attribute__((aligned(16))) char smem[];
    char *bl = smem;                                          // filters [BN][b_pitch]
    uint4 *raw = reinterpret_cast<uint4 *>(smem + a.b_bytes);  // raw tile [channel block][row][col] of VEC channels
    __shared__ int2 rowinfo[64];  // per raw row: element offset of its column 0 in X, valid flag

    const ConvTileDesc &d = a.d;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wk = wave % WAVES_K, wm = wave / WAVES_K;
    const int m0 = blockIdx.y * BN;
    const int PP = d.Ho * d.Wo;
    const T *__restrict__ X = reinterpret_cast<const T *>(a.X);
    const T *__restrict__ Wt = reinterpret_cast<const T *>(a.Wt);
    const int kg = lane >> 5, lr = lane & 31;
    const int cblocks = a.CinP / VEC;

    // ---- filters, once per workgroup: one 16-byte chunk = VEC consecutive channels of (filter, tap)
    {
        const int taps = d.KH * d.KW, per_m = taps * cblocks, chunks = BN * per_m;
        for (int c = tid; c < chunks; c += NT) {
            const int m = fast_div(c, a.magic_perm), r = c - m * per_m;
            const int tap = fast_div(r, a.magic_cb), cb = r - tap * cblocks;
            const int ky = fast_div(tap, a.magic_kw), kx = tap - ky * d.KW;
            const T *src = Wt + d.w_base + (long long)(m0 + m) * d.w_sm + ky * d.w_sy + kx * d.w_sx +
                           (long long)(cb * VEC) * d.w_sc;
            union {
                uint4 v;
                T e[VEC];
            } u;
#pragma unroll
            for (int e = 0; e < VEC; ++e)
                u.e[e] = ((m0 + m) < d.Cout && cb * VEC + e < d.Cin) ? src[(long long)e * d.w_sc] : (T)0;
            *reinterpret_cast<uint4 *>(bl + m * a.b_pitch + (tap * a.CinP + cb * VEC) * ES) = u.v;
        }
    }

    for (int tile = blockIdx.x; tile < a.tiles; tile += gridDim.x) {
        const int n0 = tile * BM;
        const int b0 = n0 / PP, y0 = (n0 - b0 * PP) / d.Wo;
        const int g0 = b0 * a.THP + y0 * d.sh;  // first raw row, counted over padded images
        if (tid < a.RR) {
            const int gr = g0 + tid, b = gr / a.THP, iy = gr - b * a.THP - d.padU;
            int2 e;
            e.y = (b < d.batch && iy >= 0 && iy < d.Hin) ? 1 : 0;
            e.x = e.y ? (int)((long long)b * d.x_sb + (long long)iy * d.x_sy) - d.padL : 0;
            rowinfo[tid] = e;
        }
        __syncthreads();  // (also: the previous tile's epilogue is done with the raw area)

        // ---- raw tile: chunk c = (cb * RR + rr) * TW + tx holds VEC channels of one input position
        {
            const int chunks = cblocks * a.PLANE;
            for (int c = tid; c < chunks; c += NT) {
                const int row = fast_div(c, a.magic_tw), tx = c - row * a.TW;
                const int cb = fast_div(row, a.magic_rr), rr = row - cb * a.RR;
                const int2 ri = rowinfo[rr];
                const int ix = tx - d.padL;
                const bool ok = ri.y && ix >= 0 && ix < d.Win;
                const T *src = X + (long long)(cb * VEC) * d.x_sc + ri.x + tx;
                union {
                    uint4 v;
                    T e[VEC];
                } u;
#pragma unroll
                for (int e = 0; e < VEC; ++e) u.e[e] = (ok && cb * VEC + e < d.Cin) ? src[(long long)e * d.x_sc] : (T)0;
                raw[c] = u.v;
            }
        }
        __syncthreads();

        // ---- contraction: tap by tap, channel blocks innermost
        int p = n0 + wm * 32 + lr;
        if (p >= a.g.N) p = a.g.N - 1;  // overhang pixels repeat the last one; they are never stored
        const int pb = p / PP, prem = p - pb * PP, py = prem / d.Wo, px = prem - py * d.Wo;
        const uint4 *arow = raw + (pb * a.THP + py * d.sh - g0) * a.TW + px * d.sw + kg * a.PLANE;
        const char *brow = bl + lr * a.b_pitch + kg * VEC * ES;

        f32x16 acc[1][FN];
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[0][j][v] = 0.f;

        const int csteps = a.CinP / KSTEP;
        int it = 0;
        for (int ky = 0; ky < d.KH; ++ky)
            for (int kx = 0; kx < d.KW; ++kx) {
                const uint4 *ap = arow + ky * a.TW + kx;
                const char *bp = brow + (ky * d.KW + kx) * a.CinP * ES;
                for (int cs = 0; cs < csteps; ++cs, ++it) {
                    if (WAVES_K > 1 && (it % WAVES_K) != wk) continue;
                    const uint4 af = ap[cs * 2 * a.PLANE];
                    uint4 bf[FN];
#pragma unroll
                    for (int j = 0; j < FN; ++j)
                        bf[j] = *reinterpret_cast<const uint4 *>(bp + j * 32 * a.b_pitch + cs * KSTEP * ES);
#pragma unroll
                    for (int j = 0; j < FN; ++j) mfma_step<T>(acc[0][j], af, bf[j]);
                }
            }
        __syncthreads();
        tile_epilogue<T, BM, BN, NT, BM / 32, 1, WAVES_K, 1, FN>(acc, a.g, reinterpret_cast<float *>(raw), a.c_mode, n0,
                                                                  m0, 0, tid, wm, 0, wk);
    }
}


template <typename T, int BM, int BN, int WAVES_K>
static int launch_conv_tile(ConvTileArgs &a, hipStream_t s) {
    constexpr int NT = (BM / 32) * WAVES_K * 64;
    auto kern = conv_tile_kernel<T, BM, BN, WAVES_K>;
    const size_t red = red_bytes<BM, BN, WAVES_K>();
    a.b_bytes = BN * a.b_pitch;
    const size_t raw_bytes = (size_t)(a.CinP / (16 / (int)sizeof(T))) * a.PLANE * 16;
    const size_t lds = (size_t)a.b_bytes + (raw_bytes > red ? raw_bytes : red);
    if (lds > 150 * 1024) return -1;
    if ((long)BN * a.d.KH * a.d.KW * (a.CinP / (16 / (int)sizeof(T))) >= 65536) return -1;
    static bool attr_set = false;
    if (!attr_set) {
        if (!hip_ok(hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, 150 * 1024),
                    "hipFuncSetAttribute"))
            return 2;
        attr_set = true;
    }
    // Persistent over pixel tiles: as many workgroups as fit on the chip at once (LDS and wave
    // slots), each walking an equal share of the tiles with its filters resident.
    a.tiles = (a.g.N + BM - 1) / BM;
    const int mt = (a.g.M + BN - 1) / BN;
    int occ = (int)((160 * 1024) / (lds + 1024));
    const int by_waves = 32 / (NT / 64);
    if (occ > by_waves) occ = by_waves;
    if (occ < 1) occ = 1;
    long cap = (long)state().num_cu * occ / mt;
    if (cap < 1) cap = 1;
    const int per_wg = (int)((a.tiles + cap - 1) / cap);
    dim3 grid((a.tiles + per_wg - 1) / per_wg, mt);
    hipLaunchKernelGGL(kern, grid, dim3(NT), lds, s, a);
    return hip_ok(hipGetLastError(), "conv tile launch") ? 0 : 2;
}

template <typename T>
int conv_tile(const ConvTileDesc &d, const void *X, const void *Wt, void *Y, const OutMap &c) {
    State &st = state();
    constexpr int ES = (int)sizeof(T), VEC = 16 / ES, KSTEP = 2 * VEC, BM = 128;
    ConvTileArgs a = {};
    a.X = X;
    a.Wt = Wt;
    a.d = d;
    a.g.C = Y;
    a.g.c = c;
    a.g.N = d.batch * d.Ho * d.Wo;
    a.g.M = d.Cout;
    a.g.K = d.Cin * d.KH * d.KW;
    a.g.splits = 1;
    a.c_mode = c_store_mode<T>(a.g);
    a.CinP = ((d.Cin + KSTEP - 1) / KSTEP) * KSTEP;
    a.THP = d.Hin + d.padU + d.padD;
    a.TW = d.Win + d.padL + d.padR;
    if (d.padU < 0 || d.padD < 0 || d.padL < 0 || d.padR < 0) return -1;
    // every output pixel's window must lie inside the padded image
    if ((d.Ho - 1) * d.sh + d.KH > a.THP || (d.Wo - 1) * d.sw + d.KW > a.TW) return -1;

    // Filters per workgroup: the narrowest of 32/64/128 that covers them (or 128 with several
    // column tiles).  The kernel pays a per-workgroup price for its filter tile, so it is only
    // used when there are pixel tiles enough to give every CU a few workgroups.
    const int bn = d.Cout <= 32 ? 32 : d.Cout <= 64 ? 64 : 128;
    const long mt = (d.Cout + bn - 1) / bn;
    if (st.gemm_path != 2 && ((long)(a.g.N + BM - 1) / BM) * mt < 2L * st.num_cu) return -1;

    // Raw rows of a tile: the output rows it spans, the image seams inside it, plus the filter height.
    const int PP = d.Ho * d.Wo;
    const int rows_spanned = (BM - 1 + d.Wo - 1) / d.Wo + 1;
    const int seams = (BM - 1 + PP - 1) / PP;
    const int seam_rows = a.THP - d.Ho * d.sh > 0 ? a.THP - d.Ho * d.sh : 0;
    a.RR = (rows_spanned - 1) * d.sh + seams * seam_rows + d.KH;
    if (a.RR > 64) return -1;
    a.PLANE = a.RR * a.TW;
    if ((long)(a.CinP / VEC) * a.PLANE >= 65536 || a.TW >= 65536) return -1;
    int pitch16 = (d.KH * d.KW * a.CinP * ES + 15) / 16;
    if ((pitch16 & 1) == 0) ++pitch16;
    a.b_pitch = pitch16 * 16;
    a.magic_tw = magic_of(a.TW);
    a.magic_rr = magic_of(a.RR);
    a.magic_perm = magic_of(d.KH * d.KW * (a.CinP / VEC));
    a.magic_cb = magic_of(a.CinP / VEC);
    a.magic_kw = magic_of(d.KW);
    // a filter tile that does not fit LDS is halved (more column tiles, each re-reading the pixels)
    int rc = -1;
    if (bn == 128) rc = launch_conv_tile<T, BM, 128, 1>(a, st.stream);
    if (rc == -1 && bn >= 64) rc = launch_conv_tile<T, BM, 64, 1>(a, st.stream);
    if (rc == -1) rc = launch_conv_tile<T, BM, 32, 1>(a, st.stream);
    return rc;
}

template int conv_tile<float>(const ConvTileDesc &, const void *, const void *, void *, const OutMap &);
template int conv_tile<half_t>(const ConvTileDesc &, const void *, const void *, void *, const OutMap &);

}  // namespace ptl
