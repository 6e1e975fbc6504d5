// 3x3 unit-stride fp16 convolution over padded positions with the input tile resident in LDS.
//
// The input arrives zero-padded and channel-blocked, xb[c/8][p] with p = (b, yp, xp) running over the padded
// grids of all samples laid end to end (16-byte chunks = 8 consecutive channels of one position), the filters
// tap-major, wr[co][tap][c].  Rows of the product are PADDED POSITIONS, not output pixels: the value of tap
// (ky, kx) for the row at position p is the chunk at p + ky*Wp + kx, so every tap is the same LDS tile read at
// a constant shift and an input element is fetched from memory once per (tile, 64-channel slab) instead of
// once per tap.  Rows whose position is not an output pixel are computed and dropped: always the last KW-1
// columns of a padded row (Wp/Wo - 1 extra work); the last KH-1 rows of every padded grid are left out of the
// row enumeration when the tile still fits (small images: rows are numbered q = (b, y < Ho, xp) and a lane's
// position is q plus (Hp - Ho)*Wp per sample boundary between the tile's first row and its own), else they
// are computed and dropped as well.
//
// A workgroup (4 waves, one per SIMD) is persistent: it walks tiles of 256 rows x BN filters.  Its work is a
// sequence of units = (tile, slab of 64 channels); a unit needs the positions of its tile plus 2*Wp + 2 for 8
// channel blocks (48 KB, two buffers: the next unit's tile is fetched while this one is used) and nine filter
// stages (tap x 64 channels x BN filters) that stream through a ring.  All loads are LDS-DMA; every wave
// issues the same number per stage, so a wait is one s_waitcnt with an immediate.  Loads past the end of the
// work re-fetch the last unit (harmless) instead of being skipped.  The immediates count only LOADS issued
// after the awaited one; result stores issued in between can only make a wait longer, never shorter.
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
    long long P;        // padded positions of all samples (stride between channel blocks of xb)
    unsigned Q;         // rows of the product
    unsigned qimg;      // rows per sample: Hp*Wp, or Ho*Wp with the bottom rows left out
    unsigned jump;      // positions skipped per sample boundary: 0 or (Hp - Ho)*Wp
    int Cin, Cout, Hp, Wp, Ho, Wo;
    int tiles, ct_count;  // tile = position tile * ct_count + filter tile
#ifdef PTL_HALO_ABL
    int abl;
#endif
};
#ifdef PTL_HALO_ABL
#define HALO_ABL(bit) (a.abl & (bit))
#else
#define HALO_ABL(bit) false
#endif

template <int I, int N, typename F>
__device__ inline void static_for(F &&f) {
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for<I + 1, N>(f);
    }
}

// ---------------------------------------------------------------------------------------------------------
// Software-pipelined form: one tap per ring stage, NS ring slots, and the landing of a stage is certified one
// stage AHEAD (wait + barrier in the middle of the stage before), so the fragment reads of k-step g + 1 can be
// issued under the MFMAs of k-step g across stage and unit boundaries: a wave never waits for LDS with an
// idle MFMA pipe except at the very start.  Slots: stage s in use, s + 1 certified, s + 2 .. s + NS - 2 in
// flight, and the slot of stage s - 1 is refilled with stage s + NS - 1 right after the barrier of stage s
// (every wave has then left stage s - 1).
template <int NS>
__host__ __device__ constexpr int pipe_pieces(int sidx) {
    // 12 tile pieces per wave and unit over the first E stages; none in the last NS - 2 stages, so that the
    // loads behind the first filter stages of a unit are the same in the prologue and in steady state
    constexpr int E = 9 - (NS - 2) < 6 ? 9 - (NS - 2) : 6;
    return sidx < E ? 12 / E + (sidx < 12 % E ? 1 : 0) : 0;
}
template <int NS>
__host__ __device__ constexpr int pipe_piece0(int sidx) {
    int n = 0;
    for (int j = 0; j < sidx; ++j) n += pipe_pieces<NS>(j);
    return n;
}
template <int NS, int LB>
__host__ __device__ constexpr int pipe_wait(int sidx) {
    // loads issued after the filters of stage sidx + 1 (issued in stage sidx - NS + 2, before that stage's pieces)
    int n = pipe_pieces<NS>((sidx - NS + 2 + 18) % 9);
    for (int j = sidx - NS + 3; j <= sidx - 1; ++j) n += LB + pipe_pieces<NS>((j + 18) % 9);
    return n;
}

template <int BN, int NS>
__global__ __launch_bounds__(HALO_NT) void conv_halo_pipe_kernel(const HaloArgs a) {
    constexpr int STAGE = BN * 128;      // bytes of a ring slot: one tap x 64 channels x BN filters
    constexpr int LB = BN / 32;          // filter chunks per thread and stage
    constexpr int FM = BN / 32, FN = 2;  // fragments per wave: filters x positions (64 positions per wave)
    constexpr int MID = 1;               // half of a stage in front of which the next stage is certified
    static_assert(NS >= 3 && NS <= 7, "ring depth");
    extern __shared__ __align__(16) char smem[];
    const unsigned halo_lds = (unsigned)(uintptr_t)(lds_char *)smem, ring_lds = halo_lds + 2 * HALO_BYTES;
    const char *const halo = smem, *const ring = smem + 2 * HALO_BYTES;
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31, kg = lane >> 5;
    const int G = gridDim.x, UC = a.Cin / 64;
    const long long K9 = 9ll * a.Cin;

    unsigned voff_b[LB];
#pragma unroll
    for (int i = 0; i < LB; ++i) {
        const int row = (wave + 4 * i) * 8 + (lane >> 3);
        voff_b[i] = (unsigned)(row * K9 * 2) + (unsigned)((((lane & 7) ^ swz(row))) << 4);
    }
    const unsigned voff_h = (unsigned)lane * 16u;
    unsigned wfrag[4];
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) wfrag[ks] = (unsigned)(l32 * 128 + (((2 * ks + kg) ^ swz(l32)) << 4));
    // byte offset of this lane's two position fragments within a tile whose first row is q0
    auto lane_offsets = [&](int tile, unsigned (&off)[FN]) {
        const unsigned q0 = (unsigned)(tile / a.ct_count) * HALO_BM, i0 = q0 / a.qimg;
#pragma unroll
        for (int j = 0; j < FN; ++j) {
            const unsigned r = (unsigned)(64 * wave + 32 * j + l32);
            const unsigned skip = a.jump ? ((q0 + r) / a.qimg - i0) * a.jump : 0u;
            off[j] = (unsigned)(kg * HALO_NP + r + skip) * 16u;
        }
    };

    auto issue_filters = [&](int tile, int cs, int tap, int slot) {
        const int ct = tile % a.ct_count;
        const char *base = a.wr + ((long long)ct * BN * K9 + (long long)tap * a.Cin + cs * 64) * 2;
        if (HALO_ABL(2)) return;
#pragma unroll
        for (int i = 0; i < LB; ++i)
            lds_dma16_saddr(voff_b[i], base, ring_lds + (unsigned)(slot * STAGE + (wave + 4 * i) * 1024));
    };
    auto issue_halo = [&](int tile, int cs, int hb, int q) {
        const unsigned q0 = (unsigned)(tile / a.ct_count) * HALO_BM;
        const long long p0 = (long long)q0 + (long long)(q0 / a.qimg) * a.jump;
        const int c0 = (q * 4 + wave) * 64, j = c0 / HALO_NP, i0 = c0 - j * HALO_NP;
        const char *base = a.xb + (((long long)(cs * 8 + j)) * a.P + p0 + i0) * 16;
        if (HALO_ABL(1)) return;
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
    auto wrap = [](int s) { return s >= NS ? s - NS : s; };

    int tile = blockIdx.x, cs = 0, hb = 0, slot = 0;  // slot: ring slot of the current stage
    int ntile, ncs;
    next_unit(tile, cs, ntile, ncs);
#pragma unroll
    for (int q = 0; q < 12; ++q) issue_halo(tile, cs, 0, q);
#pragma unroll
    for (int s = 0; s < NS - 1; ++s) issue_filters(tile, cs, s, s);  // (NS - 1 <= 9 taps: all of the first unit)
    wait_vmcnt<(NS - 2) * LB>();
    __syncthreads();  // stage 0 of the first unit has landed

    // fragment sets (two k-steps of 16 each): the one being multiplied and the one being read
    uint4 wf[2][2][FM], xf[2][2][FN];
    unsigned xoff[FN], xoff_next[FN];
    lane_offsets(tile, xoff);
    lane_offsets(ntile, xoff_next);
    auto read_frags = [&](int set, const char *wbase, const char *xtap, const unsigned (&xo)[FN], int half) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int ks = 2 * half + h;
#pragma unroll
            for (int i = 0; i < FM; ++i)
                wf[set][h][i] = *reinterpret_cast<const uint4 *>(wbase + wfrag[ks] + i * 32 * 128);
#pragma unroll
            for (int j = 0; j < FN; ++j)
                xf[set][h][j] = *reinterpret_cast<const uint4 *>(xtap + xo[j] + 2 * ks * HALO_NP * 16);
        }
    };
    read_frags(0, ring, halo, xoff, 0);

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
        const char *xbase = halo + hb * HALO_BYTES, *xnext = halo + (hb ^ 1) * HALO_BYTES;
        static_for<0, 18>([&](auto GI) {
            constexpr int g = decltype(GI)::value, sidx = g / 2, half = g % 2, cur = g & 1;
            if constexpr (half == MID) {
                // certify stage sidx + 1, then refill the slot of stage sidx - 1 with stage sidx + NS - 1
                wait_vmcnt<pipe_wait<NS, LB>(sidx)>();
                // (a bare barrier: fragment reads still in flight address slots that nobody refills now, so they
                // need not be waited for here)
                asm volatile("s_barrier" ::: "memory");
                constexpr int ahead = sidx + NS - 1;
                const int fslot = wrap(slot + NS - 1);
                if (ahead < 9)
                    issue_filters(tile, cs, ahead, fslot);
                else
                    issue_filters(ntile, ncs, ahead - 9, fslot);
                constexpr int np = pipe_pieces<NS>(sidx), q0 = pipe_piece0<NS>(sidx);
#pragma unroll
                for (int q = 0; q < np; ++q) issue_halo(ntile, ncs, hb ^ 1, q0 + q);
            }
            {  // fragments of the next pair of k-steps
                constexpr int gn = g + 1, sn = (gn / 2) % 9, hn = gn % 2;
                const int nslot = hn == 0 ? wrap(slot + 1) : slot;
                const int tapoff = ((sn / 3) * a.Wp + sn % 3) * 16;
                if (gn < 18)
                    read_frags(cur ^ 1, ring + nslot * STAGE, xbase + tapoff, xoff, hn);
                else
                    read_frags(cur ^ 1, ring + nslot * STAGE, xnext + tapoff, xoff_next, hn);
            }
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int i = 0; i < FM; ++i)
#pragma unroll
                    for (int j = 0; j < FN; ++j) mfma_step<half_t>(acc[i][j], wf[cur][h][i], xf[cur][h][j]);
            // one fragment read under each of the first MFMAs
            constexpr int R = 2 * (FM + FN), M = 2 * FM * FN;
#pragma unroll
            for (int r = 0; r < R; ++r) {
                __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            }
            if constexpr (M > R) __builtin_amdgcn_sched_group_barrier(0x008, M - R, 0);
            if (half == 1) slot = wrap(slot + 1);
        });
        const bool tile_done = cs + 1 == UC;
        if (tile_done && !HALO_ABL(4)) {
            const unsigned q0 = (unsigned)(tile / a.ct_count) * HALO_BM;
            const int co0 = (tile % a.ct_count) * BN;
            const unsigned PO = (unsigned)(a.Ho * a.Wo);
#pragma unroll
            for (int j = 0; j < FN; ++j) {
                const unsigned q = q0 + (unsigned)(64 * wave + 32 * j + l32);  // (Q < 2^31 on the host)
                const unsigned b = q / a.qimg, rem = q - b * a.qimg;
                const unsigned yy = rem / (unsigned)a.Wp, xx = rem - yy * (unsigned)a.Wp;
                if (q < a.Q && yy < (unsigned)a.Ho && xx < (unsigned)a.Wo) {
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
#pragma unroll
        for (int j = 0; j < FN; ++j) xoff[j] = xoff_next[j];
        lane_offsets(ntile, xoff_next);
    }
    wait_vmcnt<0>();  // nothing may still be landing in LDS when the workgroup ends
}

template <int BN, int NS>
int launch_halo_pipe(const HaloArgs &a, int grid, hipStream_t stream) {
    constexpr int lds = 2 * HALO_BYTES + NS * BN * 128;
    static_assert(lds <= 160 * 1024, "LDS");
    static bool attr = false;
    if (!attr) {
        if (!hip_ok(hipFuncSetAttribute((const void *)conv_halo_pipe_kernel<BN, NS>,
                                        hipFuncAttributeMaxDynamicSharedMemorySize, lds),
                    "halo convolution LDS size"))
            return 2;
        attr = true;
    }
    hipLaunchKernelGGL((conv_halo_pipe_kernel<BN, NS>), dim3((unsigned)grid), dim3(HALO_NT), lds, stream, a);
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
    // leave the bottom rows of every padded grid out when a tile that crosses sample boundaries still fits
    const int qs = d.Ho * Wp, crossings = (HALO_BM - 1 + qs - 1) / qs;
    const bool skip = Hp > d.Ho && HALO_BM + (crossings + 1) * (Hp - d.Ho) * Wp + 2 <= HALO_NP;
    a.qimg = (unsigned)(skip ? qs : Hp * Wp);
    a.jump = (unsigned)(skip ? (Hp - d.Ho) * Wp : 0);
    a.Q = (unsigned)((long long)d.batch * a.qimg);
    a.Cin = d.Cin; a.Cout = d.Cout; a.Hp = Hp; a.Wp = Wp; a.Ho = d.Ho; a.Wo = d.Wo;
    const int bn = d.Cout % 128 == 0 ? 128 : 64;
    a.ct_count = d.Cout / bn;
    const long long ptiles = ((long long)a.Q + HALO_BM - 1) / HALO_BM;
    if (ptiles * a.ct_count >= (1ll << 30)) return -1;
    a.tiles = (int)(ptiles * a.ct_count);
#ifdef PTL_HALO_ABL
    a.abl = getenv("PTL_HALO_ABL") ? atoi(getenv("PTL_HALO_ABL")) : 0;
#endif
    const int grid = a.tiles < st.num_cu ? a.tiles : st.num_cu;
    return bn == 128 ? launch_halo_pipe<128, 4>(a, grid, st.stream) : launch_halo_pipe<64, 6>(a, grid, st.stream);
}

}  // namespace ptl
