// 3x3 unit-stride fp16 convolution over padded positions with the input tile resident in LDS.
//
// The input arrives zero-padded and channel-blocked, xb[c/8][p] with p = (b, yp, xp) running over the padded
// grids of all samples laid end to end (16-byte chunks = 8 consecutive channels of one position), the filters
// tap-major, wr[co][tap][c].  Rows of the product are PADDED POSITIONS p, not output pixels: the value of tap
// (ky, kx) for row p is the chunk at p + ky*Wp + kx, so every tap is the same LDS tile read at a constant
// shift and an input element is fetched from memory once per (position tile, 64-channel slab) instead of
// once per tap.  Rows whose position is not an output pixel (the last KH-1 rows and KW-1 columns of each
// padded grid) are computed and dropped: (Hp*Wp)/(Ho*Wo) - 1 extra work.
//
// A workgroup (4 waves, one per SIMD) is persistent: it walks tiles of 256 positions x BN filters.  Its work
// is a sequence of units = (tile, slab of 64 channels); a unit needs the 256 + 2*Wp + 2 positions of its tile
// for 8 channel blocks (48 KB, two buffers: the next unit's tile is fetched while this one is used) and nine
// filter stages (tap x 64 channels x BN filters) that stream through a small ring.  All loads are LDS-DMA;
// every wave issues the same number per stage, so the wait before a stage is one s_waitcnt with an
// immediate.  Loads past the end of the work re-fetch the last unit (harmless) instead of being skipped.
// The immediates count only LOADS issued after the awaited one; result stores issued in between can only
// make a wait longer, never shorter.
#include <type_traits>

#include "ptl_conv_tile.hpp"
#include "ptl_gemm_async.hpp"
#include "ptl_gemm_async.inc"

namespace ptl {

namespace {

constexpr int HALO_BM = 256;                       // positions per tile
constexpr int HALO_NP = 384;                       // positions held per channel block (tile + 2*Wp + 2, padded)
constexpr int HALO_BYTES = HALO_NP * 8 * 16;       // one buffer: 8 channel blocks
constexpr int HALO_NT = 256;

struct HaloArgs {
    const char *xb;     // [Cin/8][P] chunks, readable HALO_NP chunks past the last tile's start in every block
    const char *wr;     // [Cout][9][Cin] halves
    half_t *y;          // [batch][Cout][Ho][Wo]
    long long P;        // padded positions of all samples
    int Cin, Cout, Hp, Wp, Ho, Wo;
    int tiles, ct_count;  // tile = position tile * ct_count + filter tile
};

// TPS taps per ring stage, NS ring slots.  Loads per thread and stage: LB filter chunks, then HP halo pieces.
template <int TPS>
__host__ __device__ constexpr int halo_pieces(int sidx) {
    // 12 pieces per wave and unit, issued early in the unit so that they are older than the first filter
    // stage of the next unit
    return TPS == 3 ? (sidx < 2 ? 6 : 0) : (sidx < 6 ? 2 : 0);
}
template <int TPS, int NS, int LB>
__host__ __device__ constexpr int halo_wait(int sidx) {
    // loads issued after those of stage sidx's filters: the halo pieces of the stage that issued them and
    // everything of the stages between
    constexpr int SU = 9 / TPS;
    int n = halo_pieces<TPS>((sidx - (NS - 1) + SU) % SU);
    for (int j = sidx - (NS - 2); j <= sidx - 1; ++j) n += LB + halo_pieces<TPS>((j + SU) % SU);
    return n;
}

template <int I, int N, typename F>
__device__ inline void static_for(F &&f) {
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for<I + 1, N>(f);
    }
}

template <int BN, int TPS, int NS>
__global__ __launch_bounds__(HALO_NT) void conv_halo_kernel(const HaloArgs a) {
    constexpr int SU = 9 / TPS;            // stages per unit
    constexpr int STAGE = TPS * BN * 128;  // bytes of a ring slot
    constexpr int LB = TPS * BN / 32;      // filter chunks per thread and stage
    constexpr int FM = BN / 32, FN = 2;    // fragments per wave: filters x positions (64 positions per wave)
    static_assert(9 % TPS == 0 && NS >= 2 && NS <= 3, "stage shape");
    extern __shared__ __align__(16) char smem[];
    const unsigned halo_lds = (unsigned)(uintptr_t)(lds_char *)smem, ring_lds = halo_lds + 2 * HALO_BYTES;
    const char *const halo = smem, *const ring = smem + 2 * HALO_BYTES;
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31, kg = lane >> 5;
    const int G = gridDim.x, UC = a.Cin / 64;
    const long long K9 = 9ll * a.Cin;

    // per-lane pieces of the addresses
    unsigned voff_b[LB];
#pragma unroll
    for (int i = 0; i < LB; ++i) {
        const int q = wave + 4 * i, tt = q / (BN / 8), row = (q % (BN / 8)) * 8 + (lane >> 3);
        voff_b[i] = (unsigned)((row * K9 + (long long)tt * a.Cin) * 2) + (unsigned)((((lane & 7) ^ swz(row))) << 4);
    }
    const unsigned voff_h = (unsigned)lane * 16u;
    unsigned wfrag[4];
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) wfrag[ks] = (unsigned)(l32 * 128 + (((2 * ks + kg) ^ swz(l32)) << 4));
    const unsigned xfrag = (unsigned)((kg * HALO_NP + 64 * wave + l32) * 16);

    auto issue_filters = [&](int tile, int cs, int sidx, int slot) {
        const int ct = tile % a.ct_count;
        const char *base = a.wr + ((long long)ct * BN * K9 + (long long)(sidx * TPS) * a.Cin + cs * 64) * 2;
#pragma unroll
        for (int i = 0; i < LB; ++i)
            lds_dma16_saddr(voff_b[i], base, ring_lds + (unsigned)(slot * STAGE + (wave + 4 * i) * 1024));
    };
    // piece q of the 12 a wave contributes to the tile of unit (tile, cs) in buffer hb
    auto issue_halo = [&](int tile, int cs, int hb, int q) {
        const long long p0 = (long long)(tile / a.ct_count) * HALO_BM;
        const int c0 = (q * 4 + wave) * 64, j = c0 / HALO_NP, i0 = c0 - j * HALO_NP;
        const char *base = a.xb + (((long long)(cs * 8 + j)) * a.P + p0 + i0) * 16;
        lds_dma16_saddr(voff_h, base, halo_lds + (unsigned)(hb * HALO_BYTES + c0 * 16));
    };
    auto next_unit = [&](int tile, int cs, int &ntile, int &ncs) {
        if (cs + 1 < UC) {
            ntile = tile;
            ncs = cs + 1;
        } else if (tile + G < a.tiles) {
            ntile = tile + G;
            ncs = 0;
        } else {  // past the end: the same unit again
            ntile = tile;
            ncs = cs;
        }
    };

    int tile = blockIdx.x, cs = 0, hb = 0, slot = 0;
    int ntile, ncs;
    next_unit(tile, cs, ntile, ncs);
    // prologue: the first unit's tile, then the first NS-1 filter stages
#pragma unroll
    for (int q = 0; q < 12; ++q) issue_halo(tile, cs, 0, q);
#pragma unroll
    for (int s = 0; s < NS - 1; ++s) issue_filters(tile, cs, s, s);

    f32x16 acc[FM][FN];
    while (true) {
        if (cs == 0) {
#pragma unroll
            for (int i = 0; i < FM; ++i)
#pragma unroll
                for (int j = 0; j < FN; ++j)
#pragma unroll
                    for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;
        }
        const char *xbase = halo + hb * HALO_BYTES + xfrag;
        static_for<0, SU>([&](auto SI) {
            constexpr int sidx = decltype(SI)::value;
            wait_vmcnt<halo_wait<TPS, NS, LB>(sidx)>();
            __syncthreads();
            {  // refill the slot stage sidx - 1 used: the filters NS - 1 stages ahead
                constexpr int ahead = sidx + NS - 1;
                int fslot = slot + NS - 1;
                if (fslot >= NS) fslot -= NS;
                if (ahead < SU)
                    issue_filters(tile, cs, ahead, fslot);
                else
                    issue_filters(ntile, ncs, ahead - SU, fslot);
                constexpr int np = halo_pieces<TPS>(sidx);
                constexpr int q0 = TPS == 3 ? 6 * sidx : 2 * sidx;
#pragma unroll
                for (int q = 0; q < np; ++q) issue_halo(ntile, ncs, hb ^ 1, q0 + q);
            }
            const char *wbase = ring + slot * STAGE;
#pragma unroll
            for (int tt = 0; tt < TPS; ++tt) {
                const int tap = sidx * TPS + tt;
                const char *xtap = xbase + ((tap / 3) * a.Wp + tap % 3) * 16;
#pragma unroll
                for (int ks = 0; ks < 4; ++ks) {
                    uint4 wf[FM], xf[FN];
#pragma unroll
                    for (int i = 0; i < FM; ++i)
                        wf[i] = *reinterpret_cast<const uint4 *>(wbase + wfrag[ks] + (tt * BN + i * 32) * 128);
#pragma unroll
                    for (int j = 0; j < FN; ++j)
                        xf[j] = *reinterpret_cast<const uint4 *>(xtap + (2 * ks * HALO_NP + j * 32) * 16);
#pragma unroll
                    for (int i = 0; i < FM; ++i)
#pragma unroll
                        for (int j = 0; j < FN; ++j) mfma_step<half_t>(acc[i][j], wf[i], xf[j]);
                }
            }
            slot = slot + 1 == NS ? 0 : slot + 1;
        });
        const bool tile_done = cs + 1 == UC;
        if (tile_done) {
            // straight from the accumulators: lane = position, four consecutive filters per register group
            const long long p0 = (long long)(tile / a.ct_count) * HALO_BM;
            const int co0 = (tile % a.ct_count) * BN;
            const unsigned plane = (unsigned)(a.Hp * a.Wp), PO = (unsigned)(a.Ho * a.Wo);
#pragma unroll
            for (int j = 0; j < FN; ++j) {
                const unsigned p = (unsigned)p0 + (unsigned)(64 * wave + 32 * j + l32);  // (P < 2^31 on the host)
                const unsigned b = p / plane, rem = p - b * plane;
                const unsigned yy = rem / (unsigned)a.Wp, xx = rem - yy * (unsigned)a.Wp;
                if (p < a.P && yy < (unsigned)a.Ho && xx < (unsigned)a.Wo) {
                    half_t *dst = a.y + ((size_t)b * a.Cout + co0 + 4 * kg) * PO + yy * (unsigned)a.Wo + xx;
#pragma unroll
                    for (int i = 0; i < FM; ++i)
#pragma unroll
                        for (int v = 0; v < 16; ++v)
                            dst[(size_t)(i * 32 + 8 * (v >> 2) + (v & 3)) * PO] = (half_t)acc[i][j][v];
                }
            }
        }
        const bool last = tile_done && tile + G >= a.tiles;
        if (last) break;
        tile = ntile;
        cs = ncs;
        hb ^= 1;
        next_unit(tile, cs, ntile, ncs);
    }
    wait_vmcnt<0>();  // nothing may still be landing in LDS when the workgroup ends
}

template <int BN, int TPS, int NS>
int launch_halo(const HaloArgs &a, int grid, hipStream_t stream) {
    constexpr int lds = 2 * HALO_BYTES + NS * TPS * BN * 128;
    static bool attr = false;
    if (!attr) {
        if (!hip_ok(hipFuncSetAttribute((const void *)conv_halo_kernel<BN, TPS, NS>,
                                        hipFuncAttributeMaxDynamicSharedMemorySize, lds),
                    "halo convolution LDS size"))
            return 2;
        attr = true;
    }
    hipLaunchKernelGGL((conv_halo_kernel<BN, TPS, NS>), dim3((unsigned)grid), dim3(HALO_NT), lds, stream, a);
    return hip_ok(hipGetLastError(), "halo convolution launch") ? 0 : 2;
}

}  // namespace

long long conv_halo_margin() { return HALO_BM + HALO_NP; }

bool conv_halo_fits(const ConvTileDesc &d, int Hp, int Wp) {
    return !d.in_hwc && d.KH == 3 && d.KW == 3 && d.sh == 1 && d.sw == 1 && d.Cin % 64 == 0 && d.Cout % 64 == 0 &&
           2 * Wp + 2 <= HALO_NP - HALO_BM && d.Ho == Hp - 2 && d.Wo == Wp - 2;
}

// xb: blocked, padded input with conv_halo_margin() readable chunks after the last block; wr: tap-major filters.
int conv_halo_launch(const ConvTileDesc &d, const void *xb, const void *wr, void *Y, int Hp, int Wp) {
    State &st = state();
    HaloArgs a = {};
    a.xb = static_cast<const char *>(xb);
    a.wr = static_cast<const char *>(wr);
    a.y = static_cast<half_t *>(Y);
    a.P = (long long)d.batch * Hp * Wp;
    a.Cin = d.Cin; a.Cout = d.Cout; a.Hp = Hp; a.Wp = Wp; a.Ho = d.Ho; a.Wo = d.Wo;
    const int bn = d.Cout % 128 == 0 ? 128 : 64;
    a.ct_count = d.Cout / bn;
    const long long ptiles = (a.P + HALO_BM - 1) / HALO_BM;
    if (ptiles * a.ct_count >= (1ll << 30)) return -1;
    a.tiles = (int)(ptiles * a.ct_count);
    const int grid = a.tiles < st.num_cu ? a.tiles : st.num_cu;
    return bn == 128 ? launch_halo<128, 1, 3>(a, grid, st.stream) : launch_halo<64, 3, 2>(a, grid, st.stream);
}

}  // namespace ptl
