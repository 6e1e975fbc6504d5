// 3x3 unit-stride fp16 convolution over padded positions with the input tile resident in LDS.
//
// The input arrives zero-padded and channel-blocked, xb[c/8][p] with p = (b, yp, xp) running over the padded
// grids of all samples laid end to end (16-byte chunks = 8 consecutive channels of one position), the filters
// tap-major, wr[co][tap][c].  Rows of the product are PADDED POSITIONS, not output pixels: the value of tap
// (ky, kx) for the row at position p is the chunk at p + ky*Wp + kx, so every tap is the same LDS tile read at
// a constant shift and an input element is fetched from memory once per (tile, 64-channel slab) instead of
// once per tap.  Rows whose position is not an output pixel are computed and dropped: the last KW-1 columns of a
// padded row (Wp/Wo - 1 extra work); the last KH-1 rows of every padded grid are left out of the row enumeration
// when the tile still fits (small images: rows are numbered q = (b, y < Ho, xp) and a lane's position is q plus
// (Hp - Ho)*Wp per sample boundary between the tile's first row and its own), else they are computed and dropped
// as well.  On narrow images, where the dropped columns are at least 1/32 of the rows, the channel-major route
// numbers its rows by OUTPUT PIXEL instead, q = (b, y, x < Wo): a lane works out its tile-local position from its
// pixel once per unit (the tile spreads over the padded grid by Wp - Wo per row boundary), nothing else changes.
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
    const char *xb;     // channel-major route: [Cin/8][P] chunks, readable HALO_NP chunks past the last tile's start in
                        // every block; channel-minor route: the tensor itself, [batch][H][W][Cin] halves
    const char *zeros;  // channel-minor route: 128 readable zero bytes
    const char *wr;     // [Cout][9][Cin] halves
    half_t *y;          // [batch][Cout][Ho][Wo], channel-minor route [batch][Ho][Wo][Cout]
    long long P;        // padded positions of all samples (stride between channel blocks of xb)
    unsigned Q;         // rows of the product
    unsigned qimg;      // rows per sample: Hp*Wp, or Ho*Wp with the rows below the sample left out
    unsigned jump;      // positions skipped per sample boundary: 0 or (Hp - Ho)*Wp
    unsigned maxcross;  // sample boundaries a tile can cross (0 when jump is 0)
    unsigned m_img, m_row;  // channel-minor route: multipliers for position / (Hp*Wp) and / Wp (see fast_div31)
    int s_img, s_row;
    int batch, Cin, Cout, Hp, Wp, Ho, Wo;
    int tiles, ct_count;  // tile = position tile * ct_count + filter tile
    int xcd_map;          // 1: the grid is a multiple of 8 and a workgroup's first tile follows its XCD
    // channel-major route, optional: the output once more as the next layer's blocked, padded input
    half_t *yblk;           // [Cout/8][yb_P] chunks of eight filters, nullptr: no such copy
    unsigned yb_P;          // chunks per block of eight filters: batch * yb_Hp * yb_Wp
    int yb_Hp, yb_Wp, yb_padU, yb_padL;
    int yb_relu;            // 1: the copy holds max(output, 0)
    // channel-major route: rows are output pixels (b, y, x < Wo) instead of padded positions (b, y, xp < Wp): no row of
    // the product is a dropped column, and consecutive rows are consecutive pixels of the output
    int dense;
    unsigned m_wo;          // multiplier and shift for / Wo (see fast_div31)
    int s_wo;
    unsigned row_lim;       // dense: largest tile-local position a row may have (rows past the end are clamped to it)
};

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

// The products run on v_mfma_f32_16x16x32_f16: a fragment is 16 rows x 32 k (a lane holds row lane % 16, k group
// lane / 16 of eight), one ds_read_b128 each as with the 32 x 32 x 16 form and the same bytes from LDS per flop; a
// lane then holds four consecutive filters of one position.  These kernels run against the board's power limit (on
// random operands the clock drops until the power fits), and there the 16 x 16 x 32 form sustains more: a loop of
// nothing but MFMAs 1.9 against 1.7 PFLOP/s, this kernel 4-9 % on 512 -> 512 channels measured on one board in turns.
__device__ inline void mfma16(f32x4 &acc, const uint4 &a, const uint4 &b) {
    acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), acc, 0, 0, 0);
}

// n / d for n < 2^31 with m = ceil(2^(31 + s) / d), s = ceil(log2 d) >= 1 (d >= 2)
__device__ inline unsigned fast_div31(unsigned n, unsigned m, int s) { return __umulhi(n, m) >> (s - 1); }

// Everything about a unit that the loads of its stages need, worked out once per unit (wave-uniform).
struct HaloUnit {
    int tile, cs;
    const char *fb;   // filters of (filter tile, channel slab): + tap * Cin * 2 per stage, + voff_b per lane
    const char *hb;   // channel-major: this wave's first input piece (blocks 2 * wave and 2 * wave + 1 of the slab, from
                      // the tile's first position); channel-minor: the tensor + the slab's byte offset in a pixel
    unsigned p0;      // position of the tile's first row in the padded grids laid end to end
    unsigned rem0;    // row of the tile's first position within its sample's rows
    unsigned loc0;    // dense rows: padded position of the tile's first row within its sample's grid
};

// HWC = false: the input arrives zero-padded and channel-blocked (see the head of the file).
// HWC = true: channel-minor tensors read in place.  X[b][y][x][c] already consists of the 16-byte chunks the
// kernel wants, the 64 channels of a slab are 128 consecutive bytes of a pixel, and the filters W[co][ky][kx][ci]
// of the forward pass are tap-major as they lie.  What is missing is the zero border - and that costs nothing,
// because every lane of a load gives its own address: the input tile in LDS is a run of positions of a VIRTUAL
// padded grid with ONE zero row above and ONE zero column left of every sample,
//     V[b][yv][xv] = X[b][yv - 1][xv - 1]  for yv, xv >= 1,   zero for yv = 0 or xv = 0 or b >= batch,
// Hp = H + 1 rows of Wp = W + 1 columns: the column right of a row's last pixel is the zero column of the next row,
// the row below a sample's last row the zero row of the next sample.  A lane whose position is a zero of the grid
// loads from a page of zeros.  So a layer is ONE launch and only one column in Wp (and, where the row below a
// sample is not skipped, one row in Hp) is computed and dropped.  The tile in LDS is then [position][8 chunks] (a
// wave's load covers 8 positions x 128 bytes: whole cache lines), the chunks of a row XOR-swizzled like the filter
// rows, and a fragment address is (row << 7) + ((chunk << 4) ^ swizzle(row)) with the tap's shift inside `row`.
template <int BN, int NS, bool HWC>
__global__ __launch_bounds__(HALO_NT) void conv_halo_kernel(const HaloArgs a) {
    constexpr int STAGE = BN * 128;      // bytes of a ring slot: one tap x 64 channels x BN filters
    constexpr int LB = BN / 32;          // filter chunks per thread and stage
    constexpr int FM = BN / 16, FN = 4;  // fragments per wave: filters x positions (64 positions per wave)
    constexpr int MID = 1;               // half of a stage in front of which the next stage is certified
    constexpr int NR = FM + FN, NM = FM * FN;  // fragment reads / MFMAs per half stage (one k-step of 32)
    static_assert(NS >= 3 && NS <= 7, "ring depth");
    extern __shared__ __align__(16) char smem[];
    const unsigned halo_lds = (unsigned)(uintptr_t)(lds_char *)smem, ring_lds = halo_lds + 2 * HALO_BYTES;
    const char *const halo = smem, *const ring = smem + 2 * HALO_BYTES;
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l16 = lane & 15, kq = lane >> 4;
    const int G = gridDim.x, UC = a.Cin / 64;
    const long long K9 = 9ll * a.Cin, P16 = a.P * 16;
    const int cin2 = a.Cin * 2;
    const unsigned HpWp = (unsigned)(a.Hp * a.Wp);

    unsigned voff_b[LB];
#pragma unroll
    for (int i = 0; i < LB; ++i) {
        const int row = (wave + 4 * i) * 8 + (lane >> 3);
        voff_b[i] = (unsigned)(row * K9 * 2) + (unsigned)((((lane & 7) ^ swz(row))) << 4);
    }
    const unsigned voff_h = (unsigned)lane * 16u;
    unsigned wfrag[2];
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) wfrag[ks] = (unsigned)(l16 * 128 + (((4 * ks + kq) ^ swz(l16)) << 4));

    // The divisions that locate a tile and the 64-bit products behind its addresses are about a hundred scalar
    // instructions: once per unit, not once per load.
    auto make_unit = [&](int tile, int cs) {
        HaloUnit u;
        u.tile = tile;
        u.cs = cs;
        const unsigned pt = (unsigned)tile / (unsigned)a.ct_count, ct = (unsigned)tile - pt * (unsigned)a.ct_count;
        const unsigned q0 = pt * HALO_BM, b0 = q0 / a.qimg;
        u.rem0 = q0 - b0 * a.qimg;
        u.p0 = q0 + b0 * a.jump;  // (the host keeps the positions, a tile's reach included, below 2^31)
        u.loc0 = 0;
        if (!HWC && a.dense) {
            const unsigned y0 = u.rem0 / (unsigned)a.Wo, x0 = u.rem0 - y0 * (unsigned)a.Wo;
            u.loc0 = y0 * (unsigned)a.Wp + x0;
            u.p0 = b0 * HpWp + u.loc0;
        }
        u.fb = a.wr + ((long long)ct * BN * K9 + cs * 64) * 2;
        u.hb = HWC ? a.xb + cs * 128 : a.xb + ((long long)(cs * 8 + 2 * wave) * a.P + u.p0) * 16;
        return u;
    };
    // tile-local position of the row of this lane's fragment j: its row number plus `jump` per sample boundary
    // between the tile's first row and its own
    auto lane_rows = [&](const HaloUnit &u, unsigned (&row)[FN]) {
#pragma unroll
        for (int j = 0; j < FN; ++j) {
            const unsigned r = (unsigned)(64 * wave + 16 * j + l16), v = u.rem0 + r;
            if (!HWC && a.dense) {
                // pixel (cross samples on, y, x) -> its padded position, from the tile's first one
                unsigned cross = 0;
                for (unsigned k = 1, lim = a.qimg; k <= a.maxcross; ++k, lim += a.qimg) cross += v >= lim ? 1u : 0u;
                const unsigned w = v - cross * a.qimg;
                const unsigned y = fast_div31(w, a.m_wo, a.s_wo), x = w - y * (unsigned)a.Wo;
                row[j] = min(cross * HpWp + y * (unsigned)a.Wp + x - u.loc0, a.row_lim);
                continue;
            }
            unsigned skip = 0;
            for (unsigned k = 1, lim = a.qimg; k <= a.maxcross; ++k, lim += a.qimg) skip += v >= lim ? a.jump : 0u;
            row[j] = r + skip;
        }
    };
    auto next_unit = [&](const HaloUnit &u) {
        if (u.cs + 1 < UC) return make_unit(u.tile, u.cs + 1);
        if (u.tile + G < a.tiles) return make_unit(u.tile + G, 0);
        return u;  // past the end: the same unit again
    };
    // load i of a filter stage / piece q (0 .. 11) of a unit's input tile
    auto issue_filter = [&](const HaloUnit &u, int tap, unsigned slot_lds, int i) {
        lds_dma16_saddr(voff_b[i], u.fb + tap * cin2, slot_lds + (unsigned)((wave + 4 * i) * 1024));
    };
    auto issue_piece = [&](const HaloUnit &u, unsigned buf_lds, int q) {
        if constexpr (HWC) {
            // eight positions x the slab's eight chunks per wave and piece
            const unsigned pl = (unsigned)((wave + 4 * q) * 8 + (lane >> 3));  // tile-local position
            const unsigned pv = u.p0 + pl;
            const unsigned b = fast_div31(pv, a.m_img, a.s_img), rem = pv - b * HpWp;
            const unsigned yv = fast_div31(rem, a.m_row, a.s_row), xv = rem - yv * (unsigned)a.Wp;
            const bool ok = b < (unsigned)a.batch && yv >= 1u && xv >= 1u;
            const unsigned chunk = (unsigned)(((lane & 7) ^ swz((int)pl)) << 4);
            const unsigned pix = (b * (unsigned)a.Ho + yv - 1u) * (unsigned)a.Wo + xv - 1u;  // < 2^31 / Cin
            const char *src = ok ? u.hb + ((size_t)pix * (unsigned)cin2 + chunk) : a.zeros + chunk;
            lds_dma<16>(src, buf_lds + (unsigned)((wave + 4 * q) * 1024));
        } else {
            // pieces 0..5: block 2 * wave, pieces 6..11: block 2 * wave + 1; 64 positions each
            const char *base = u.hb + (q >= 6 ? P16 : 0ll) + (q % 6) * 1024;
            lds_dma16_saddr(voff_h, base, buf_lds + (unsigned)(((2 * wave + q / 6) * HALO_NP + (q % 6) * 64) * 16));
        }
    };

    // Workgroups are dealt to the 8 XCDs in turn, each with an L2 of its own: XCD x takes the tiles [x * G/8, (x+1) * G/8)
    // of every round, so that the filter tiles of one position tile - neighbours in the tile order, readers of the same
    // input tile - and position tiles that overlap in their reach meet in one L2.
    const int first_tile = a.xcd_map ? (int)(blockIdx.x & 7) * (G >> 3) + (int)(blockIdx.x >> 3) : (int)blockIdx.x;
    HaloUnit cu = make_unit(first_tile, 0), nu = next_unit(cu);
    int hb = 0;
    unsigned slot_off = 0, prev_off = (NS - 1) * STAGE;  // ring slot of the current stage / of the stage before it
#pragma unroll
    for (int q = 0; q < 12; ++q) issue_piece(cu, halo_lds, q);
#pragma unroll
    for (int s = 0; s < NS - 1; ++s)  // (NS - 1 <= 9 taps: all of the first unit)
#pragma unroll
        for (int i = 0; i < LB; ++i) issue_filter(cu, s, ring_lds + s * STAGE, i);
    wait_vmcnt<(NS - 2) * LB>();
    __syncthreads();  // stage 0 of the first unit has landed

    // fragment sets (one k-step of 32 each): the one being multiplied and the one being read
    uint4 wf[2][FM], xf[2][FN];
    unsigned xrow[FN], xrow_next[FN];
    lane_rows(cu, xrow);
    lane_rows(nu, xrow_next);
    // per position fragment j of the tap being read: channel-major, the byte offset of (k group, row) in a tile whose
    // channel blocks are HALO_NP chunks apart; channel-minor, (row << 7) and the swizzle term of the row
    unsigned xa[FN], xt[FN];
    auto tap_addresses = [&](const unsigned (&row)[FN], int shift) {
#pragma unroll
        for (int j = 0; j < FN; ++j) {
            const unsigned rt = row[j] + (unsigned)shift;
            if constexpr (HWC) {
                xa[j] = rt << 7;
                xt[j] = ((rt << 3) & 0x70u) ^ (unsigned)(kq << 4);
            } else {
                xa[j] = (unsigned)(kq * HALO_NP + rt) * 16u;
            }
        }
    };
    // read r (0 .. NR - 1) of the fragments of k-step ks of a stage, in the order the MFMAs first need them: the first
    // filter fragment, the position fragments, the other filter fragments
    auto read_frag = [&](int set, const char *wbase, const char *xbuf, int ks, int r) {
        if (r == 0 || r > FN) {
            const int i = r == 0 ? 0 : r - FN;
            wf[set][i] = *reinterpret_cast<const uint4 *>(wbase + wfrag[ks] + i * 16 * 128);
        } else if constexpr (HWC) {
            xf[set][r - 1] = *reinterpret_cast<const uint4 *>(xbuf + (xa[r - 1] + (xt[r - 1] ^ (unsigned)(ks << 6))));
        } else {
            xf[set][r - 1] = *reinterpret_cast<const uint4 *>(xbuf + xa[r - 1] + 4 * ks * HALO_NP * 16);
        }
    };
    tap_addresses(xrow, 0);
#pragma unroll
    for (int r = 0; r < NR; ++r) read_frag(0, ring, halo, 0, r);

    f32x4 acc[FM][FN];
    while (true) {
        if (cu.cs == 0) {
#pragma unroll
            for (int i = 0; i < FM; ++i)
#pragma unroll
                for (int j = 0; j < FN; ++j)
#pragma unroll
                    for (int v = 0; v < 4; ++v) acc[i][j][v] = 0.f;
        }
        const char *xbase = halo + hb * HALO_BYTES, *xnext = halo + (hb ^ 1) * HALO_BYTES;
        const unsigned next_lds = halo_lds + (unsigned)((hb ^ 1) * HALO_BYTES);
        static_for<0, 18>([&](auto GI) {
            constexpr int g = decltype(GI)::value, sidx = g / 2, half = g % 2, cur = g & 1;
            // loads this half stage issues: the filters of stage sidx + NS - 1 into the slot of stage sidx - 1, then
            // this stage's share of the next unit's input tile
            constexpr int ahead = sidx + NS - 1;
            constexpr int np = half == MID ? pipe_pieces<NS>(sidx) : 0, q0 = pipe_piece0<NS>(sidx);
            constexpr int nd = half == MID ? LB + np : 0;
            // (the 32-filter tile has two MFMAs behind its six fragment reads: its loads go two to an MFMA)
            constexpr int per = nd > NM - NR ? (nd + NM - NR - 1) / (NM - NR) : 1;  // loads behind one MFMA
            constexpr int dstep = per > 1 ? 1 : (NM - NR) / (nd > 0 ? nd : 1);     // MFMAs between two loads
            static_assert(dstep >= 1, "fragment reads first, then the loads spread over the other MFMAs");
            if constexpr (half == MID) {
                // certify stage sidx + 1; every wave has then left stage sidx - 1
                wait_vmcnt<pipe_wait<NS, LB>(sidx)>();
                // (a bare barrier: fragment reads still in flight address slots that nobody refills now, so they
                // need not be waited for here)
                asm volatile("s_barrier" ::: "memory");
            }
            // fragments of the next k-step
            constexpr int gn = g + 1, sn = (gn / 2) % 9, hn = gn % 2;
            const unsigned noff = hn == 0 ? (slot_off + STAGE == NS * STAGE ? 0u : slot_off + STAGE) : slot_off;
            const char *wnext = ring + noff, *xbuf = gn < 18 ? xbase : xnext;
            if constexpr (hn == 0) {  // a new tap (of the next unit's tile behind the last stage)
                const int shift = (sn / 3) * a.Wp + sn % 3;
                if constexpr (gn < 18)
                    tap_addresses(xrow, shift);
                else
                    tap_addresses(xrow_next, shift);
            }
            // One fragment read behind each of the first MFMAs, then the loads spread over the others, in exactly this
            // order (nothing may cross a sched_barrier): the address arithmetic of a load sits between two MFMAs
            // instead of in front of a run of them.
            static_for<0, NM>([&](auto MI) {
                constexpr int m = decltype(MI)::value, i = m / FN, j = m % FN;
                if constexpr (m < NR) read_frag(cur ^ 1, wnext, xbuf, hn, m);
                mfma16(acc[i][j], wf[cur][i], xf[cur][j]);
                if constexpr (m >= NR && (m - NR) % dstep == 0) {
                    static_for<0, per>([&](auto PI) {
                        constexpr int d = (m - NR) / dstep * per + decltype(PI)::value;
                        if constexpr (d < nd) {
                            if constexpr (d < LB) {
                                if constexpr (ahead < 9)
                                    issue_filter(cu, ahead, ring_lds + prev_off, d);
                                else
                                    issue_filter(nu, ahead - 9, ring_lds + prev_off, d);
                            } else {
                                issue_piece(nu, next_lds, q0 + d - LB);
                            }
                        }
                    });
                }
                __builtin_amdgcn_sched_barrier(0);
            });
            if constexpr (half == 1) {
                prev_off = slot_off;
                slot_off = slot_off + STAGE == NS * STAGE ? 0u : slot_off + STAGE;
            }
        });
        const bool tile_done = cu.cs + 1 == UC;
        if (tile_done) {
            const unsigned q0 = ((unsigned)cu.tile / (unsigned)a.ct_count) * HALO_BM;
            const int co0 = (cu.tile % a.ct_count) * BN;
            const unsigned PO = (unsigned)(a.Ho * a.Wo);
            if constexpr (HWC) {
#pragma unroll
                for (int j = 0; j < FN; ++j) {
                    const unsigned q = q0 + (unsigned)(64 * wave + 16 * j + l16);  // (Q < 2^31 on the host)
                    const unsigned b = q / a.qimg, rem = q - b * a.qimg;
                    const unsigned yy = rem / (unsigned)a.Wp, xx = rem - yy * (unsigned)a.Wp;
                    if (q < a.Q && yy < (unsigned)a.Ho && xx < (unsigned)a.Wo) {
                        // a lane holds four consecutive filters of its position per filter fragment
                        half_t *dst = a.y + ((size_t)b * PO + yy * (unsigned)a.Wo + xx) * (unsigned)a.Cout + co0 + 4 * kq;
#pragma unroll
                        for (int i = 0; i < FM; ++i) {
                            union {
                                half_t e[4];
                                uint2 v;
                            } o;
#pragma unroll
                            for (int v = 0; v < 4; ++v) o.e[v] = (half_t)acc[i][j][v];
                            *reinterpret_cast<uint2 *>(dst + i * 16) = o.v;
                        }
                    }
                }
            } else {
                // Channel-major output: a row of 16 lanes holds four consecutive filters of 16 positions per fragment,
                // which as it stands is four 32-byte runs per store.  The four position fragments (registers) and
                // the four filter groups (rows of lanes) change places - two swaps of lane rows per register, on
                // the values already rounded to halves and packed in pairs - so that lane l holds position l of
                // the wave's 64 and every filter of the tile: a store is then one run of 128 bytes, and the copy
                // for the next layer one 16-byte chunk per lane and eight filters.
                typedef unsigned pk_t;
                pk_t pk[FM][FN][2];
#pragma unroll
                for (int i = 0; i < FM; ++i)
#pragma unroll
                    for (int j = 0; j < FN; ++j)
#pragma unroll
                        for (int h = 0; h < 2; ++h) {
                            union {
                                half_t e[2];
                                pk_t u;
                            } o;
                            o.e[0] = (half_t)acc[i][j][2 * h];
                            o.e[1] = (half_t)acc[i][j][2 * h + 1];
                            pk[i][j][h] = o.u;
                        }
                static_assert(FN == 4, "four position fragments against four rows of lanes");
#pragma unroll
                for (int i = 0; i < FM; ++i)
#pragma unroll
                    for (int h = 0; h < 2; ++h) {
                        const auto s01 = __builtin_amdgcn_permlane16_swap(pk[i][0][h], pk[i][1][h], false, false);
                        const auto s23 = __builtin_amdgcn_permlane16_swap(pk[i][2][h], pk[i][3][h], false, false);
                        const auto t02 = __builtin_amdgcn_permlane32_swap(s01[0], s23[0], false, false);
                        const auto t13 = __builtin_amdgcn_permlane32_swap(s01[1], s23[1], false, false);
                        pk[i][0][h] = t02[0];  // now [i][kk][h]: filters i*16 + 4*kk + 2*h, + 1 of position `lane`
                        pk[i][2][h] = t02[1];
                        pk[i][1][h] = t13[0];
                        pk[i][3][h] = t13[1];
                    }
                const unsigned q = q0 + (unsigned)(64 * wave + lane);  // (Q < 2^31 on the host)
                const unsigned b = q / a.qimg, rem = q - b * a.qimg;
                const unsigned rw = a.dense ? (unsigned)a.Wo : (unsigned)a.Wp;  // rows of the enumeration are this wide
                const unsigned yy = rem / rw, xx = rem - yy * rw;
                if (q < a.Q && yy < (unsigned)a.Ho && xx < (unsigned)a.Wo) {
                    half_t *dst = a.y + ((size_t)b * a.Cout + co0) * PO + yy * (unsigned)a.Wo + xx;
#pragma unroll
                    for (int i = 0; i < FM; ++i)
#pragma unroll
                        for (int kk = 0; kk < 4; ++kk)
#pragma unroll
                            for (int h = 0; h < 2; ++h) {
                                union {
                                    half_t e[2];
                                    pk_t u;
                                } o;
                                o.u = pk[i][kk][h];
                                dst[(size_t)(i * 16 + 4 * kk + 2 * h) * PO] = o.e[0];
                                dst[(size_t)(i * 16 + 4 * kk + 2 * h + 1) * PO] = o.e[1];
                            }
                    if (a.yblk) {
                        const unsigned pos = ((b * (unsigned)a.yb_Hp + yy + (unsigned)a.yb_padU) * (unsigned)a.yb_Wp) + xx +
                                             (unsigned)a.yb_padL;
#pragma unroll
                        for (int i = 0; i < FM; ++i)
#pragma unroll
                            for (int c = 0; c < 2; ++c) {
                                const unsigned cb = (unsigned)(co0 + i * 16 + 8 * c) >> 3;
                                uint4 ch = make_uint4(pk[i][2 * c][0], pk[i][2 * c][1], pk[i][2 * c + 1][0], pk[i][2 * c + 1][1]);
                                if (a.yb_relu) {
                                    typedef _Float16 h2_t __attribute__((ext_vector_type(2)));
                                    const h2_t z = {(_Float16)0, (_Float16)0};
                                    auto pos2 = [&](unsigned u) {
                                        return __builtin_bit_cast(unsigned, __builtin_elementwise_max(__builtin_bit_cast(h2_t, u), z));
                                    };
                                    ch = make_uint4(pos2(ch.x), pos2(ch.y), pos2(ch.z), pos2(ch.w));
                                }
                                *reinterpret_cast<uint4 *>(a.yblk + ((size_t)cb * a.yb_P + pos) * 8) = ch;
                            }
                    }
                }
            }
        }
        const bool last = tile_done && cu.tile + G >= a.tiles;
        if (last) break;
        cu = nu;
        hb ^= 1;
        nu = next_unit(cu);
#pragma unroll
        for (int j = 0; j < FN; ++j) xrow[j] = xrow_next[j];
        lane_rows(nu, xrow_next);
    }
    wait_vmcnt<0>();  // nothing may still be landing in LDS when the workgroup ends
}

template <int BN, int NS, bool HWC>
int launch_halo(const HaloArgs &a, int grid, hipStream_t stream) {
    constexpr int lds = 2 * HALO_BYTES + NS * BN * 128;
    static_assert(lds <= 160 * 1024, "LDS");
    static bool attr = false;
    if (!attr) {
        if (!hip_ok(hipFuncSetAttribute((const void *)conv_halo_kernel<BN, NS, HWC>,
                                        hipFuncAttributeMaxDynamicSharedMemorySize, lds),
                    "halo convolution LDS size"))
            return 2;
        attr = true;
    }
    hipLaunchKernelGGL((conv_halo_kernel<BN, NS, HWC>), dim3((unsigned)grid), dim3(HALO_NT), lds, stream, a);
    return hip_ok(hipGetLastError(), "halo convolution launch") ? 0 : 2;
}


// ---------------------------------------------------------------------------------------------------------
// Weight gradient on the same layouts:
//   dW[co][ci][ky][kx] = sum over padded positions p of  gb[p][co] * xb[p + ky*Wp + kx][ci]
// with gb the output gradient embedded at the top left of the padded grids (zero elsewhere), channel-blocked
// like xb.  The contraction runs over positions, so both operands sit in LDS as [position][8 channels] chunks
// and a fragment is two transposing reads (ds_read_b64_tr_b16); a tap is a shift by whole chunks, so every
// read stays aligned.  A workgroup (4 waves) owns 128 filters x 64 channels x a group of taps (0..4 or 5..8)
// and a range of positions; it walks units of 128 positions (gradient tile 32 KB, two buffers; input tile of the
// 192 positions that the taps reach when the rows are at most 31 wide, else 256, of which consecutive units share
// all but 128: a ring, see HWG_RING; the next unit in flight while this one is multiplied) with all accumulators in
// registers
// and writes one fp32 partial sum per tap at the end; a second kernel adds the partial sums.
constexpr int HWG_UNIT = 128;                 // positions per unit
constexpr int HWG_GP = 132, HWG_XP = 260;     // LDS pitches (chunks) of the gradient / input tiles: == 4 mod 16,
                                              // so that the 16 rows of a transposing read fall on distinct banks
constexpr int HWG_GB = 16 * HWG_GP * 16, HWG_XB = 8 * HWG_XP * 16, HWG_BUF = HWG_GB + HWG_XB;
// Channel-major form: the input tiles of consecutive units overlap (unit u reads positions 128 u .. 128 u + 64 R - 1,
// R = 3 or 4 pieces of 64), so they live in ONE ring of six 64-position slots per channel block, piece j in slot
// j % 6, behind the two gradient buffers; a unit brings in two new pieces.  Slots 6 and 7 repeat slots 0 and 1 (a
// piece that lands in slot 0, or in slot 1 when R = 4, is loaded a second time there), so the reads of a unit, which
// start at slot 0, 2 or 4, never wrap.
constexpr int HWG_RP = 8 * 64 + 4, HWG_RB = 8 * HWG_RP * 16, HWG_RING = 2 * HWG_GB;

struct HaloWgArgs {
    const char *xb;    // [Cin/8][Px] chunks, readable 256 chunks past the start of the last unit
    const char *gb;    // [Cout/8][Pd] chunks, Pd a multiple of HWG_UNIT, zero from the last padded position on
    float *ws;         // partial sums [tap][smax][Cout][Cin]
    long long Px, Pd;
    int Cin, Cout, Wp;
    int units;         // Pd / HWG_UNIT
    int tiles_ci;      // Cin / 64
    int tiles;         // (Cout / 128) * (Cin / 64)
    int S0, S1, smax;  // position splits of the two tap groups
    int xcd_map;       // 1: bundles of `tiles` workgroups per XCD (see the kernel)
    int x_pieces;      // 64-position pieces of the input tile that the taps can reach: 3 when 2 * Wp + 2 <= 64, else 4
    // channel-minor tensors read in place (HWC = true): xb = X[batch][H][W][Cin], gb = dY[batch][H][W][Cout]
    const char *zeros;
    int batch, H, W, Hp;
    unsigned m_img, m_row;
    int s_img, s_row;
};

typedef short hwg_s4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) hwg_s4 hwg_lds_s4;

// A fragment = two transposing reads, `second` bytes (four positions) apart.
__device__ inline uint4 hwg_frag(const char *p, int second) {
    union {
        hwg_s4 h[2];
        uint4 v;
    } t;
    t.h[0] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((hwg_lds_s4 *)(lds_char *)p);
    t.h[1] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((hwg_lds_s4 *)(lds_char *)(p + second));
    return t.v;
}

// HWC = true: the tiles filled from channel-minor tensors where they lie.  The positions are those of the virtual
// grid of the forward kernel (one zero row above and one zero column left of every sample, Hp = H + 1 rows of
// Wp = W + 1 positions): position (b, yv, xv) of the gradient tile is dY[b][yv][xv] for yv < H and xv < W, of the
// input tile X[b][yv - 1][xv - 1] for yv, xv >= 1 - the pixel of the gradient tile Wp + 1 positions earlier - and a
// chunk of zeros otherwise.  So ONE table of 256 pixel indices per unit (-1: zeros), entry e = the gradient-tile
// pixel of position p0 - (Wp + 1) + e, serves both tiles; a thread works out one entry (two multiply-shift
// divisions), a unit ahead, into one of two slots behind the tile buffers.  The tiles are [position][chunk] in
// LDS - a load covers whole 128-byte runs of the tensors: 8 positions x 8 chunks of the input tile, 4 positions x
// 16 chunks of the gradient tile - with the chunks of a position rotated by two slots per position, which puts
// the 16 pieces of a transposing read (4 positions x 2 channel blocks x 2 halves) on 16 different 8-byte cells of
// one 128-byte stripe; a lane's channel block in a load and its offsets in the fragment reads do not depend on
// the unit, the tap shift is part of the per-tap offset.
// FI: 16-filter blocks per wave: 4 = 128 filters per workgroup (two tap groups of 5 and 4 taps), 2 = 64 filters
// (all nine taps in one workgroup).
template <int T0, int NT, bool HWC, int FI>
__device__ inline void halo_wg_body(const HaloWgArgs &a, char *smem, int tile, int split, int S) {
    const unsigned lds0 = (unsigned)(uintptr_t)(lds_char *)smem;
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave & 1, wn = wave >> 1;
    const int i16 = lane & 15, kq = lane >> 4;
    const int co_cb0 = (tile / a.tiles_ci) * (4 * FI), ci_cb0 = (tile % a.tiles_ci) * 8;
    const int u0 = (int)((long long)split * a.units / S), u1 = (int)((long long)(split + 1) * a.units / S);
    const unsigned voff = (unsigned)lane * 16u;
    static_assert(HWC || FI == 4, "the channel-major form has 128-filter tiles only");

    // ---- channel-minor: position table and loads
    int *const tab = reinterpret_cast<int *>(smem + 2 * HWG_BUF);
    auto fill_table = [&](int u, int slot) {
        const long long pt = (long long)u * HWG_UNIT - (a.Wp + 1) + tid;
        int v = -1;
        if (pt >= 0) {
            const unsigned pv = (unsigned)pt, HpWp = (unsigned)(a.Hp * a.Wp);
            const unsigned b = fast_div31(pv, a.m_img, a.s_img), rem = pv - b * HpWp;
            const unsigned yv = fast_div31(rem, a.m_row, a.s_row), xv = rem - yv * (unsigned)a.Wp;
            if (b < (unsigned)a.batch && yv < (unsigned)a.H && xv < (unsigned)a.W)
                v = (int)((b * (unsigned)a.H + yv) * (unsigned)a.W + xv);  // (the host keeps pixel counts below 2^31)
        }
        tab[slot * 256 + tid] = v;
    };
    // this lane's channel block in every load of the gradient / input tile, as a byte offset within a pixel
    const unsigned g_chunk = (unsigned)(co_cb0 + (((lane & 15) & 8) | (((lane & 7) - 2 * (lane >> 4)) & 7))) * 16u;
    const unsigned x_chunk = (unsigned)(ci_cb0 + (((lane & 7) - 2 * (lane >> 3)) & 7)) * 16u;
    const unsigned cout2 = (unsigned)a.Cout * 2u, cin2 = (unsigned)a.Cin * 2u;
    auto issue_hwc = [&](int buf, int slot) {
        const int *t = tab + slot * 256;
        constexpr int GQ = 2 * FI;  // loads of the gradient tile per wave: 128 positions x 4 * FI chunks
#pragma unroll
        for (int q = 0; q < 8; ++q) {
            if (q < GQ) {
                // 64 / (4 * FI) positions x 4 * FI chunks per load
                constexpr int PPL = 16 / FI;  // positions per load
                const int ig = wave * GQ + q;
                const int idx = t[ig * PPL + (FI == 4 ? lane >> 4 : lane >> 3) + a.Wp + 1];
                const unsigned chunk = FI == 4 ? g_chunk : (unsigned)(co_cb0 + (((lane & 7) - 2 * (lane >> 3)) & 7)) * 16u;
                const char *src = idx >= 0 ? a.gb + ((size_t)(unsigned)idx * cout2 + chunk) : a.zeros;
                lds_dma<16>(src, lds0 + (unsigned)(buf * HWG_BUF + ig * 1024));
            }
            if (wave < a.x_pieces) {  // (wave w loads positions 64 w .. 64 w + 63 of the input tile)
                const int ix = wave * 8 + q;
                const int idx = t[ix * 8 + (lane >> 3)];
                const char *src = idx >= 0 ? a.xb + ((size_t)(unsigned)idx * cin2 + x_chunk) : a.zeros;
                lds_dma<16>(src, lds0 + (unsigned)(buf * HWG_BUF + HWG_GB + ix * 1024));
            }
        }
    };

    // 64 positions of input channel block cb, from position pos on, into slot `slot` of the ring
    auto issue_x = [&](long long pos, int cb, int slot) __attribute__((always_inline)) {
        const char *base = a.xb + ((long long)(ci_cb0 + cb) * a.Px + pos) * 16;
        lds_dma16_saddr(voff, base, lds0 + (unsigned)(HWG_RING + (cb * HWG_RP + slot * 64) * 16));
    };
    // the gradient tile of unit u into buffer buf and, first = true: the R pieces of its input tile into slots 0 ..
    // R - 1 (wave w loads piece w); else, k3 = (u - 1 - u0) % 3: its two last pieces, (u - u0) * 2 + R - 2 and the next
    auto issue = [&](int u, int buf, bool first, int k3) __attribute__((always_inline)) {
        const long long p0 = (long long)u * HWG_UNIT;
#pragma unroll
        for (int q = 0; q < 8; ++q) {  // gradient tile: 16 channel blocks x 2 pieces of 64 positions
            const int idx = q * 4 + wave, cb = idx >> 1, piece = idx & 1;
            const char *base = a.gb + ((long long)(co_cb0 + cb) * a.Pd + p0 + piece * 64) * 16;
            lds_dma16_saddr(voff, base, lds0 + (unsigned)(buf * HWG_GB + (cb * HWG_GP + piece * 64) * 16));
        }
        if (first) {
            if (wave < a.x_pieces) {
#pragma unroll
                for (int cb = 0; cb < 8; ++cb) issue_x(p0 + wave * 64, cb, wave);
            }
        } else {
            const int R = a.x_pieces, pc = wave & 1;
            int slot = 2 * k3 + R + pc;
            slot = slot >= 6 ? slot - 6 : slot;
            const long long pos = p0 + (R - 2 + pc) * 64;
#pragma unroll
            for (int q = 0; q < 4; ++q) issue_x(pos, q * 2 + (wave >> 1), slot);
            if (slot < R - 2) {
#pragma unroll
                for (int q = 0; q < 4; ++q) issue_x(pos, q * 2 + (wave >> 1), slot + 6);
            }
        }
    };

    // A wave owns 16 * FI filters x 32 channels x NT taps as 16 x 16 blocks (v_mfma_f32_16x16x32_f16: 32 positions per
    // k-step, a lane holds row lane % 16 and positions 8 * (lane / 16) .. + 7 of the step).  This lane's piece of a
    // transposing read: position k0 + i16 / 4 of channel block .. + (i16 & 3) / 2, channels 4 * (i16 & 1) .. + 3 of
    // that block; the second read of a fragment is four positions on.
    // Byte offsets of this lane's first read of gradient fragment i / input fragment (c, tap) in k-step 0; a k-step on is
    // + KSG / KSX bytes, the second read + RDG / RDX.
    constexpr int GROW = HWC ? (FI == 4 ? 256 : 128) : 16;  // bytes from one position of the gradient tile to the next
    constexpr int KSG = 32 * GROW, RDG = 4 * GROW, KSX = HWC ? 32 * 128 : 512, RDX = HWC ? 4 * 128 : 64;
    const int pj = (i16 & 3) >> 1, pq = i16 >> 2, ph = (i16 & 1) * 8;
    unsigned goff[FI], xoff[2][NT];
#pragma unroll
    for (int i = 0; i < FI; ++i) {
        if constexpr (HWC) {
            const int cb = wm * 2 * FI + 2 * i + pj;  // block within the tile's 4 * FI
            goff[i] = (unsigned)((8 * kq + pq) * GROW + ((cb & 8) | (((cb & 7) + 2 * pq) & 7)) * 16 + ph);
        } else {
            goff[i] = (unsigned)((((wm * 8 + 2 * i + pj) * HWG_GP + 8 * kq + pq) * 16) + ph);
        }
    }
#pragma unroll
    for (int c = 0; c < 2; ++c)
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            const int sh = ((T0 + t) / 3) * a.Wp + (T0 + t) % 3;
            if constexpr (HWC)
                xoff[c][t] = (unsigned)(HWG_GB + (8 * kq + pq + sh) * 128 + ((wn * 4 + 2 * c + pj + 2 * pq + 2 * sh) & 7) * 16 + ph);
            else
                xoff[c][t] = (unsigned)(HWG_RING + (((wn * 4 + 2 * c + pj) * HWG_RP + 8 * kq + pq + sh) * 16) + ph);
        }

    f32x4 acc[FI][2][NT];
#pragma unroll
    for (int i = 0; i < FI; ++i)
#pragma unroll
        for (int c = 0; c < 2; ++c)
#pragma unroll
            for (int t = 0; t < NT; ++t)
#pragma unroll
                for (int v = 0; v < 4; ++v) acc[i][c][t][v] = 0.f;

    if (u0 < u1) {
        if constexpr (HWC) {
            fill_table(u0, 0);
            __syncthreads();
            issue_hwc(0, 0);
            if (u0 + 1 < u1) fill_table(u0 + 1, 1);
        } else {
            issue(u0, 0, true, 0);
        }
    }
    int k3 = 0;  // (u - u0) % 3: the unit's input tile starts at slot 2 * k3 of the ring
    for (int u = u0; u < u1; ++u) {
        const int buf = (u - u0) & 1;
        wait_vmcnt<0>();
        __syncthreads();  // unit u has landed for every wave, and every wave has left unit u - 1
        if constexpr (HWC) {
            // the table of unit u + 1 was written before the barrier; that of unit u + 2 takes the slot of unit u,
            // whose loads were issued before the barrier
            if (u + 1 < u1) issue_hwc(buf ^ 1, buf ^ 1);
            if (u + 2 < u1) fill_table(u + 2, buf);
        } else {
            if (u + 1 < u1) issue(u + 1, buf ^ 1, false, k3);
        }
        const char *bt = smem + buf * (HWC ? HWG_BUF : HWG_GB);
        const char *xt = HWC ? bt : smem + k3 * (2 * 64 * 16);
        k3 = k3 == 2 ? 0 : k3 + 1;
        uint4 gf[2][FI], xf[2][2][NT];
        auto read = [&](int set, int ks) {
#pragma unroll
            for (int i = 0; i < FI; ++i) gf[set][i] = hwg_frag(bt + goff[i] + ks * KSG, RDG);
#pragma unroll
            for (int c = 0; c < 2; ++c)
#pragma unroll
                for (int t = 0; t < NT; ++t) xf[set][c][t] = hwg_frag(xt + xoff[c][t] + ks * KSX, RDX);
        };
        read(0, 0);
        static_for<0, 4>([&](auto KI) {
            constexpr int ks = decltype(KI)::value, cur = ks & 1;
            if constexpr (ks + 1 < 4) read(cur ^ 1, ks + 1);
#pragma unroll
            for (int i = 0; i < FI; ++i)
#pragma unroll
                for (int c = 0; c < 2; ++c)
#pragma unroll
                    for (int t = 0; t < NT; ++t) mfma16(acc[i][c][t], gf[cur][i], xf[cur][c][t]);
            if constexpr (ks + 1 < 4) {
                // 2 * (FI + 2 * NT) transposing reads under 2 * FI * NT MFMAs: one read (two where the reads outnumber
                // the MFMAs) behind each of the first MFMAs
                constexpr int RD = 2 * (FI + 2 * NT), MF = 2 * FI * NT, PER = (RD + MF - 1) / MF;
#pragma unroll
                for (int m = 0; m < (RD + PER - 1) / PER; ++m) {
                    __builtin_amdgcn_sched_group_barrier(0x100, PER, 0);
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                }
            }
        });
    }
    wait_vmcnt<0>();  // nothing may still be landing in LDS when the workgroup ends
    if (u0 >= u1) return;
    // partial sums: lane = channel, four consecutive filters per block
    const int co0 = (tile / a.tiles_ci) * (32 * FI) + wm * (16 * FI) + 4 * kq, ci0 = (tile % a.tiles_ci) * 64 + wn * 32 + i16;
#pragma unroll
    for (int t = 0; t < NT; ++t) {
        float *dst = a.ws + (((size_t)(T0 + t) * a.smax + split) * a.Cout + co0) * a.Cin + ci0;
#pragma unroll
        for (int i = 0; i < FI; ++i)
#pragma unroll
            for (int c = 0; c < 2; ++c)
#pragma unroll
                for (int v = 0; v < 4; ++v) dst[(size_t)(i * 16 + v) * a.Cin + c * 16] = acc[i][c][t][v];
    }
}

template <bool HWC, int FI>
__global__ __launch_bounds__(HALO_NT) void conv_halo_wg_kernel(const HaloWgArgs a) {
    extern __shared__ __align__(16) char smem[];
    // The workgroups of one (tap group, position split) - one per tile of the weight tensor - stream the same
    // positions at the same time: the gradient tile is read by the tiles of a filter block, the input tile by the
    // tiles of a channel block.  Workgroups are dealt to the 8 XCDs in turn, so such a bundle takes every eighth
    // workgroup: its tiles meet in one L2 (measured on 256 -> 256 channels, 28x28, batch 256: 9.4 M of the kernel's
    // 14.5 M L2 requests missed with the bundles spread over the XCDs, 3.9 M this way; the run time did not change -
    // the kernel runs against the board's power limit, not against its memory).
    int tile, bundle;
    if (a.xcd_map) {
        const int xcd = blockIdx.x & 7, j = blockIdx.x >> 3;
        tile = j % a.tiles;
        bundle = (j / a.tiles) * 8 + xcd;
        if (bundle >= a.S0 + a.S1) return;
    } else {
        const int id = blockIdx.x, n0 = a.tiles * a.S0;
        tile = id < n0 ? id / a.S0 : (id - n0) / a.S1;
        bundle = id < n0 ? id % a.S0 : a.S0 + (id - n0) % a.S1;
    }
    if constexpr (FI == 2) {
        halo_wg_body<0, 9, HWC, 2>(a, smem, tile, bundle, a.S0);  // (64-filter tiles: one group of nine taps, S1 = 0)
    } else {
        if (bundle < a.S0)
            halo_wg_body<0, 5, HWC, 4>(a, smem, tile, bundle, a.S0);
        else
            halo_wg_body<5, 4, HWC, 4>(a, smem, tile, bundle - a.S0, a.S1);
    }
}

// dW[idx * 9 + tap] (filters [co][ci][tap]) or, tap-major, dW[((idx / Cin) * 9 + tap) * Cin + idx % Cin] (filters
// [co][tap][ci]) = sum over the splits of the tap's group of ws[tap][split][idx], idx = co * Cin + ci
__global__ __launch_bounds__(256) void conv_halo_wg_reduce_kernel(const float *__restrict__ ws, half_t *__restrict__ dW,
                                                                  long long total, int S0, int S1, int smax,
                                                                  int tap_major_cin) {
    // 64 outputs x 4 groups of splits per workgroup (a 64 x 64 filter tensor still gives 576 workgroups), four loads
    // in flight per thread, the four groups added in a fixed order
    __shared__ float part[4][64];
    const int o = threadIdx.x & 63, sg = threadIdx.x >> 6, tap = blockIdx.y;
    const long long idx = (long long)blockIdx.x * 64 + o;
    const int S = tap < 5 ? S0 : S1;
    float s = 0.f;
    if (idx < total) {
        const float *src = ws + (size_t)tap * smax * total + idx;
        int z = sg;
        for (; z + 12 < S; z += 16) {
            float v[4];
#pragma unroll
            for (int k = 0; k < 4; ++k) v[k] = src[(size_t)(z + 4 * k) * total];
            s += (v[0] + v[1]) + (v[2] + v[3]);
        }
        for (; z < S; z += 4) s += src[(size_t)z * total];
    }
    part[sg][o] = s;
    __syncthreads();
    if (sg != 0 || idx >= total) return;
    s = (part[0][o] + part[1][o]) + (part[2][o] + part[3][o]);
    if (tap_major_cin > 0)
        dW[((idx / tap_major_cin) * 9 + tap) * tap_major_cin + idx % tap_major_cin] = (half_t)s;
    else
        dW[idx * 9 + tap] = (half_t)s;
}

// The same sums, in the same order, for four consecutive outputs per thread (16-byte loads); total % 4 == 0 and, where
// the filters are tap-major, tap_major_cin % 4 == 0.
__global__ __launch_bounds__(256) void conv_halo_wg_reduce4_kernel(const float *__restrict__ ws, half_t *__restrict__ dW,
                                                                   long long total, int S0, int S1, int smax,
                                                                   int tap_major_cin) {
    __shared__ float4 part[4][64];
    const int o = threadIdx.x & 63, sg = threadIdx.x >> 6, tap = blockIdx.y;
    const long long idx = ((long long)blockIdx.x * 64 + o) * 4;
    const int S = tap < 5 ? S0 : S1;
    float4 s = make_float4(0.f, 0.f, 0.f, 0.f);
    if (idx < total) {
        const float *src = ws + (size_t)tap * smax * total + idx;
        auto ld = [&](int z) { return *reinterpret_cast<const float4 *>(src + (size_t)z * total); };
        int z = sg;
        for (; z + 12 < S; z += 16) {
            float4 v[4];
#pragma unroll
            for (int k = 0; k < 4; ++k) v[k] = ld(z + 4 * k);
            s.x += (v[0].x + v[1].x) + (v[2].x + v[3].x);
            s.y += (v[0].y + v[1].y) + (v[2].y + v[3].y);
            s.z += (v[0].z + v[1].z) + (v[2].z + v[3].z);
            s.w += (v[0].w + v[1].w) + (v[2].w + v[3].w);
        }
        for (; z < S; z += 4) {
            const float4 v = ld(z);
            s.x += v.x; s.y += v.y; s.z += v.z; s.w += v.w;
        }
    }
    part[sg][o] = s;
    __syncthreads();
    if (sg != 0 || idx >= total) return;
    const float4 p0 = part[0][o], p1 = part[1][o], p2 = part[2][o], p3 = part[3][o];
    const float r[4] = {(p0.x + p1.x) + (p2.x + p3.x), (p0.y + p1.y) + (p2.y + p3.y), (p0.z + p1.z) + (p2.z + p3.z),
                        (p0.w + p1.w) + (p2.w + p3.w)};
    if (tap_major_cin > 0) {
        union {
            half_t e[4];
            uint2 v;
        } out;
#pragma unroll
        for (int k = 0; k < 4; ++k) out.e[k] = (half_t)r[k];
        *reinterpret_cast<uint2 *>(dW + ((idx / tap_major_cin) * 9 + tap) * tap_major_cin + idx % tap_major_cin) = out.v;
    } else {
#pragma unroll
        for (int k = 0; k < 4; ++k) dW[(idx + k) * 9 + tap] = (half_t)r[k];
    }
}

// Channel-major filters [co][ci][tap], many outputs: the nine taps of an output are nine 2-byte stores 18 bytes apart
// from nine workgroups in the kernels above (21 M such stores for 512 x 512 filters: 8 of the 14 us of that
// addition).  Here a workgroup adds all nine taps of 256 consecutive outputs - the same sums in the same order, a
// thread's loads of the nine taps in flight together - and writes their 4608 bytes in 16-byte pieces.
// total % 256 == 0.
__global__ __launch_bounds__(256) void conv_halo_wg_reduce9_kernel(const float *__restrict__ ws, half_t *__restrict__ dW,
                                                                   long long total, int S0, int S1, int smax) {
    __shared__ float4 part[9][4][64];
    __shared__ __align__(16) half_t outv[256 * 9];
    const int o = threadIdx.x & 63, sg = threadIdx.x >> 6;
    const long long idx = ((long long)blockIdx.x * 64 + o) * 4;
    float4 s[9];
#pragma unroll
    for (int tap = 0; tap < 9; ++tap) {
        const int S = tap < 5 ? S0 : S1;
        const float *src = ws + (size_t)tap * smax * total + idx;
        auto ld = [&](int z) { return *reinterpret_cast<const float4 *>(src + (size_t)z * total); };
        s[tap] = make_float4(0.f, 0.f, 0.f, 0.f);
        int z = sg;
        for (; z + 12 < S; z += 16) {
            float4 v[4];
#pragma unroll
            for (int k = 0; k < 4; ++k) v[k] = ld(z + 4 * k);
            s[tap].x += (v[0].x + v[1].x) + (v[2].x + v[3].x);
            s[tap].y += (v[0].y + v[1].y) + (v[2].y + v[3].y);
            s[tap].z += (v[0].z + v[1].z) + (v[2].z + v[3].z);
            s[tap].w += (v[0].w + v[1].w) + (v[2].w + v[3].w);
        }
        for (; z < S; z += 4) {
            const float4 v = ld(z);
            s[tap].x += v.x; s[tap].y += v.y; s[tap].z += v.z; s[tap].w += v.w;
        }
    }
#pragma unroll
    for (int tap = 0; tap < 9; ++tap) part[tap][sg][o] = s[tap];
    __syncthreads();
    // wave sg: taps sg, sg + 4 (and 8 for wave 0) of the quads
    for (int tap = sg; tap < 9; tap += 4) {
        const float4 p0 = part[tap][0][o], p1 = part[tap][1][o], p2 = part[tap][2][o], p3 = part[tap][3][o];
        const float r[4] = {(p0.x + p1.x) + (p2.x + p3.x), (p0.y + p1.y) + (p2.y + p3.y), (p0.z + p1.z) + (p2.z + p3.z),
                            (p0.w + p1.w) + (p2.w + p3.w)};
#pragma unroll
        for (int k = 0; k < 4; ++k) outv[(o * 4 + k) * 9 + tap] = (half_t)r[k];
    }
    __syncthreads();
    uint4 *dst = reinterpret_cast<uint4 *>(dW + (long long)blockIdx.x * 256 * 9);
    for (int j = threadIdx.x; j < 256 * 9 * 2 / 16; j += 256) dst[j] = reinterpret_cast<const uint4 *>(outv)[j];
}

// gb[cb][p] for p < pstride (see halo_embed_chunk).
__global__ __launch_bounds__(256) void conv_halo_embed_kernel(const half_t *__restrict__ dy, uint4 *__restrict__ out,
                                                              int B, int Ho, int Wo, int Hp, int Wp, int pu, int pl,
                                                              long long sb, long long sc, unsigned P, unsigned pstride,
                                                              unsigned total) {
    const unsigned i = blockIdx.x * 256u + threadIdx.x;
    if (i < total) halo_embed_chunk(i, dy, out, Ho, Wo, Hp, Wp, pu, pl, sb, sc, P, pstride);
}

}  // namespace

long long conv_halo_margin() { return HALO_BM + HALO_NP; }

bool conv_halo_fits(const ConvTileDesc &d, int Hp, int Wp) {
    return !d.in_hwc && d.KH == 3 && d.KW == 3 && d.sh == 1 && d.sw == 1 && d.Cin % 64 == 0 && d.Cout % 32 == 0 &&
           2 * Wp + 2 <= HALO_NP - HALO_BM && conv_output_fits_pads(d) && Hp >= d.Ho && Wp >= d.Wo;
}

static void magic31(unsigned d, unsigned *m, int *s);

// xb: blocked, padded input with conv_halo_margin() readable chunks after the last block; wr: tap-major filters.
int conv_halo_launch(const ConvTileDesc &d, const void *xb, const void *wr, void *Y, int Hp, int Wp, long long pstride,
                     const HaloOutCopy *oc) {
    State &st = state();
    HaloArgs a = {};
    a.xb = static_cast<const char *>(xb);
    a.wr = static_cast<const char *>(wr);
    a.y = static_cast<half_t *>(Y);
    a.P = pstride > 0 ? pstride : (long long)d.batch * Hp * Wp;
    if (a.P + HALO_NP >= ((long long)1 << 31)) return -1;
    // leave the bottom rows of every padded grid out when a tile that crosses sample boundaries still fits
    const int qs = d.Ho * Wp, crossings = (HALO_BM - 1 + qs - 1) / qs;
    // (a tile's positions: its rows, the rows skipped at the boundaries it crosses, and its reach of two rows and two
    // positions)
    const bool skip = Hp > d.Ho && HALO_BM + crossings * (Hp - d.Ho) * Wp + 2 * Wp + 2 <= HALO_NP;
    a.qimg = (unsigned)(skip ? qs : Hp * Wp);
    a.jump = (unsigned)(skip ? (Hp - d.Ho) * Wp : 0);
    a.maxcross = (unsigned)(skip ? crossings : 0);
    // rows = output pixels where the tile and its reach still fit: a tile's 256 pixels spread over the padded grid by
    // Wp - Wo per row boundary and by the rows left out per sample boundary
    // (where the dropped columns are at least a thirty-second of the rows: below that - 56 x 56 images - the per-lane
    // division costs more than they do, 41.5 against 40.4 us on 64 -> 64 channels at batch 128)
    for (int leave = 1; leave >= 0 && !a.dense && d.Wo >= 2 && (Wp - d.Wo) * 32 >= Wp; --leave) {
        const int rows = leave ? d.Ho : Hp;  // rows of a sample in the enumeration
        if (leave && Hp == d.Ho) continue;
        const int qd = rows * d.Wo, cross = (HALO_BM - 1 + qd - 1) / qd;
        const int spread = ((d.Wo + HALO_BM - 2) / d.Wo) * (Wp - d.Wo) + cross * (Hp - rows) * Wp;
        if (HALO_BM + spread + 2 * Wp + 2 > HALO_NP) continue;
        a.dense = 1;
        a.qimg = (unsigned)qd;
        a.jump = 0;
        a.maxcross = (unsigned)cross;
        a.row_lim = (unsigned)(HALO_NP - 2 * Wp - 3);
        magic31((unsigned)d.Wo, &a.m_wo, &a.s_wo);
    }
    a.Q = (unsigned)((long long)d.batch * a.qimg);
    a.batch = d.batch; a.Cin = d.Cin; a.Cout = d.Cout; a.Hp = Hp; a.Wp = Wp; a.Ho = d.Ho; a.Wo = d.Wo;
    if (oc && oc->buf) {
        // every output pixel must land inside the copy's grid, and the copy's chunks are counted in 32 bits
        const long long plane = (long long)d.batch * oc->Hp * oc->Wp;
        if (oc->padU < 0 || oc->padL < 0 || d.Ho + oc->padU > oc->Hp || d.Wo + oc->padL > oc->Wp || d.Cout % 8 != 0 ||
            plane * (d.Cout / 8) >= ((long long)1 << 31))
            return -1;
        a.yblk = static_cast<half_t *>(oc->buf);
        a.yb_P = (unsigned)plane;
        a.yb_Hp = oc->Hp; a.yb_Wp = oc->Wp; a.yb_padU = oc->padU; a.yb_padL = oc->padL;
        a.yb_relu = oc->relu;
    }
    const int bn = d.Cout % 128 == 0 ? 128 : d.Cout % 64 == 0 ? 64 : 32;
    a.ct_count = d.Cout / bn;
    const long long ptiles = ((long long)a.Q + HALO_BM - 1) / HALO_BM;
    if (ptiles * a.ct_count >= (1ll << 30)) return -1;
    a.tiles = (int)(ptiles * a.ct_count);
    const int grid = a.tiles < st.num_cu ? a.tiles : st.num_cu;
    a.xcd_map = grid % 8 == 0;
    return bn == 128  ? launch_halo<128, 4, false>(a, grid, st.stream)
           : bn == 64 ? launch_halo<64, 6, false>(a, grid, st.stream)
                      : launch_halo<32, 7, false>(a, grid, st.stream);
}

// Channel-minor 3x3 "same" layers (one row / column of padding on every side), unit stride, whole 64-channel slabs
// on both sides, rows short enough for a tile and its reach to fit the LDS buffer, 16-byte aligned tensors.
bool conv_halo_hwc_fits(const ConvTileDesc &d, const void *X, const void *Y) {
    const int Wv = d.Win + 1;
    return d.in_hwc && d.KH == 3 && d.KW == 3 && d.sh == 1 && d.sw == 1 && d.padU == 1 && d.padD == 1 && d.padL == 1 &&
           d.padR == 1 && d.Ho == d.Hin && d.Wo == d.Win && d.Cin % 64 == 0 && d.Cout % 64 == 0 && d.Cin <= 8192 &&
           HALO_BM + 2 * Wv + 2 <= HALO_NP && reinterpret_cast<uintptr_t>(X) % 16 == 0 &&
           reinterpret_cast<uintptr_t>(Y) % 8 == 0 &&
           (long long)(d.batch + 1) * (d.Hin + 1) * Wv + HALO_NP < ((long long)1 << 31);
}

static void magic31(unsigned d, unsigned *m, int *s) {  // d >= 2
    int l = 1;
    while ((1ull << l) < d) ++l;
    *s = l;
    *m = (unsigned)(((1ull << (31 + l)) + d - 1) / d);
}

// X: [batch][H][W][Cin], wr: tap-major filters [Cout][9][Cin], Y: [batch][H][W][Cout].
int conv_halo_hwc_launch(const ConvTileDesc &d, const void *X, const void *wr, void *Y) {
    State &st = state();
    HaloArgs a = {};
    a.xb = static_cast<const char *>(X);
    a.zeros = static_cast<const char *>(st.zeros);
    a.wr = static_cast<const char *>(wr);
    a.y = static_cast<half_t *>(Y);
    a.batch = d.batch; a.Cin = d.Cin; a.Cout = d.Cout; a.Ho = d.Hin; a.Wo = d.Win;
    a.Hp = d.Hin + 1; a.Wp = d.Win + 1;
    // leave the zero row of every sample out of the row enumeration when a tile that crosses sample boundaries and
    // its reach (two rows and two positions) still fit
    const int qs = d.Hin * a.Wp, crossings = (HALO_BM - 1 + qs - 1) / qs;
    const bool skip = HALO_BM + crossings * a.Wp + 2 * a.Wp + 2 <= HALO_NP;
    a.qimg = (unsigned)(skip ? qs : a.Hp * a.Wp);
    a.jump = (unsigned)(skip ? a.Wp : 0);
    a.maxcross = (unsigned)(skip ? crossings : 0);
    a.Q = (unsigned)((long long)d.batch * a.qimg);
    magic31((unsigned)(a.Hp * a.Wp), &a.m_img, &a.s_img);
    magic31((unsigned)a.Wp, &a.m_row, &a.s_row);
    const int bn = d.Cout % 128 == 0 ? 128 : 64;
    a.ct_count = d.Cout / bn;
    const long long ptiles = ((long long)a.Q + HALO_BM - 1) / HALO_BM;
    if (ptiles * a.ct_count >= (1ll << 30)) return -1;
    a.tiles = (int)(ptiles * a.ct_count);
    const int grid = a.tiles < st.num_cu ? a.tiles : st.num_cu;
    a.xcd_map = grid % 8 == 0;
    return bn == 128 ? launch_halo<128, 4, true>(a, grid, st.stream) : launch_halo<64, 6, true>(a, grid, st.stream);
}

bool conv_halo_wg_fits(const ConvTileDesc &d, int Hp, int Wp) {
    return !d.in_hwc && d.KH == 3 && d.KW == 3 && d.sh == 1 && d.sw == 1 && d.Cin % 64 == 0 && d.Cout % 128 == 0 &&
           2 * Wp + 2 <= 128 && conv_output_fits_pads(d) && Hp >= d.Ho && Wp >= d.Wo &&
           (long long)d.batch * Hp * Wp < ((long long)1 << 31);
}
// Measured against the alternatives (fp16): at batch 128..512, 128 -> 128 on 28x28 73 / 243 against 87 / 306 us
// (resident output tile kernel), 256 -> 256 on 14x14 70 against 83 us and on 28x28 384 against 390 us, 512 -> 512 on
// 7x7 69 against 86 us (tap-sum GEMM); from 256 channels it wins from 20 units of positions on (512 -> 512 on 7x7 at
// batch 32: 38 against 53 us; 256 -> 256 on 14x14 at batch 8, 16 units: 30 against 26 us for the resident output tile
// kernel), with 128 channels only from about a hundred (128 -> 128 on 14x14 at batch 32: 28
// against 25 us for the resident output tile kernel).  (Measured before the input tiles of consecutive units shared a
// ring; the starting points below are from after.)
bool conv_halo_wg_preferred(const ConvTileDesc &d) {
    int Hp, Wp;
    conv_padded_grid(d, &Hp, &Wp);
    const long long units = ((long long)d.batch * Hp * Wp + HWG_UNIT - 1) / HWG_UNIT;
    const int cmin = d.Cin < d.Cout ? d.Cin : d.Cout;
    // Rows 33 to 63 wide (four pieces of the input tile per unit; the ring made them cheaper), against the routes they
    // took before, in turns in one process: 128 -> 128 on 56x56 at batch 128 205 against 237 us (batch 8: 30.0 / 32.2),
    // 128 -> 256 on 56x56 at batch 64 178 / 233, on 48x48 at batch 128 267 / 355, 256 -> 256 on 32x32 at batch 128
    // 202 / 222 (batch 16: 40.6 / 56.0, batch 4: equal), on 56x56 at batch 64 319 / 330, 128 -> 128 on 40x40 at
    // batch 256 207 / 223 (batch 8: 24.9 / 30.7); with 64 channels 64 -> 128 on 56x56 at batch 128 132 / 137, at
    // batch 16 equal, at batch 4 23.4 against 20.6: those only from 1600 units on.
    const bool wide_ok = Wp <= 32 || cmin >= 128 || units >= 1600;
    // Where it starts to pay, in units of 128 positions (this route against the one chosen without it, in turns in one
    // process): 512 -> 512 on 14x14 from 14 (batch 8: 35.5 against 39.8 us; batch 4, 7 units: 34.3 / 30.2); 256 -> 256
    // from 20 (14x14 at batch 8, 14 units: 30.7 / 25.7); 128 channels on a side from 48 (128 -> 128 on 28x28 at batch
    // 8, 52 units: 24.3 / 28.6; batch 4, 26 units: 21.5 / 15.0), from 28 with four and more tiles of the filter tensor
    // (128 -> 256 on 14x14 at batch 16: 26.1 / 35.8).
    const int tiles = (d.Cout / 128) * (d.Cin / 64);
    const long long need = cmin >= 512 ? 14 : cmin >= 256 ? 20 : cmin >= 128 ? (tiles >= 4 ? 28 : 48) : 96;
    return conv_halo_wg_fits(d, Hp, Wp) && wide_ok && units >= need;
}
// Channel-minor: the other route copies both tensors into padded form first (9 + 9 of 66 us on 128 -> 128 28x28 at
// batch 128), so this one is taken from the same amount of work on whatever the row length.
bool conv_halo_wg_hwc_preferred(const ConvTileDesc &d) {
    const long long units = ((long long)d.batch * (d.Hin + 1) * (d.Win + 1) + HWG_UNIT - 1) / HWG_UNIT;
    const int cmin = d.Cin < d.Cout ? d.Cin : d.Cout;
    // the same starting points as for the channel-major form, measured the same way: 512 -> 512 on 14x14 at batch 8
    // 33.4 against 51.0 us, 128 -> 128 on 28x28 at batch 8 / 12 22.9 / 23.5 against 26.9 / 35.5 (batch 4: 18.3 / 14.5),
    // 128 -> 256 on 14x14 at batch 16 24.8 / 26.6, 256 -> 256 on 14x14 at batch 8 (14 units) 27.8 / 23.6
    const int tiles = ((d.Cout + 127) / 128) * (d.Cin / 64);
    return units >= (cmin >= 512 ? 14 : cmin >= 256 ? 20 : cmin >= 128 ? (tiles >= 4 ? 28 : 48) : 96);
}
long long conv_halo_wg_margin() { return 2 * HWG_UNIT + 256; }
long long conv_halo_wg_gradient_stride(const ConvTileDesc &d, int Hp, int Wp) {
    const long long P = (long long)d.batch * Hp * Wp;
    return (P + HWG_UNIT - 1) / HWG_UNIT * HWG_UNIT;
}
size_t conv_halo_wg_partial_bytes(const ConvTileDesc &d, int Hp, int Wp, int *S0, int *S1) {
    State &st = state();
    const long long units = conv_halo_wg_gradient_stride(d, Hp, Wp) / HWG_UNIT;
    if (d.Cout % 128) {  // 64-filter tiles (channel-minor only): all nine taps in one workgroup, one split count
        const int tiles = (d.Cout / 64) * (d.Cin / 64);
        long long s = st.num_cu / tiles;
        if (s < 1) s = 1;
        if (s > units) s = units;
        *S0 = (int)s;
        *S1 = (int)s;
        return (size_t)9 * s * d.Cout * d.Cin * sizeof(float);
    }
    const int tiles = (d.Cout / 128) * (d.Cin / 64);
    // one workgroup per CU; the two tap groups (five and four taps) get position splits in the ratio 5 : 4 so that
    // their workgroups finish together
    long long per_tile = st.num_cu / tiles;
    if (per_tile < 2) per_tile = 2;
    long long s0 = (per_tile * 5 + 4) / 9, s1 = per_tile - s0;
    if (s1 < 1) s1 = 1;
    if (s0 > units) s0 = units;
    if (s1 > units) s1 = units;
    *S0 = (int)s0;
    *S1 = (int)s1;
    const long long smax = s0 > s1 ? s0 : s1;
    return (size_t)9 * smax * d.Cout * d.Cin * sizeof(float);
}

// A channel-major tensor t[batch][C][Hs][Ws] as padded, channel-blocked chunks out[C / 8][pstride] (see
// conv_halo_embed_kernel): the tensor sits pu rows / pl columns inside each Hp x Wp grid.
int conv_halo_embed(const void *t, void *out, int batch, int C, int Hs, int Ws, int Hp, int Wp, int pu, int pl,
                    long long pstride) {
    State &st = state();
    const long long P = (long long)batch * Hp * Wp, chunks = (long long)(C / 8) * pstride;
    if (chunks >= ((long long)1 << 31) || pstride < P) return -1;
    hipLaunchKernelGGL(conv_halo_embed_kernel, dim3((unsigned)((chunks + 255) / 256)), dim3(256), 0, st.stream,
                       static_cast<const half_t *>(t), static_cast<uint4 *>(out), batch, Hs, Ws, Hp, Wp, pu, pl,
                       (long long)C * Hs * Ws, (long long)Hs * Ws, (unsigned)P, (unsigned)pstride, (unsigned)chunks);
    return hip_ok(hipGetLastError(), "blocked layout launch") ? 0 : 2;
}

template <bool HWC, int FI>
static int halo_wg_run(HaloWgArgs &a, const ConvTileDesc &d, float *ws, void *dW) {
    State &st = state();
    // channel-minor: two buffers of both tiles + the two position tables; channel-major: two gradient buffers + the ring
    constexpr int lds = HWC ? 2 * HWG_BUF + 2 * 256 * (int)sizeof(int) : HWG_RING + HWG_RB;
    static bool attr = false;
    if (!attr) {
        if (!hip_ok(hipFuncSetAttribute((const void *)conv_halo_wg_kernel<HWC, FI>,
                                        hipFuncAttributeMaxDynamicSharedMemorySize, lds),
                    "halo weight-gradient LDS size"))
            return 2;
        attr = true;
    }
    a.xcd_map = 1;
    // the last tap reads positions up to 127 + 2 * Wp + 2 of the input tile: within its first 192 for rows up to 31 wide
    a.x_pieces = 2 * a.Wp + 2 <= 64 ? 3 : 4;
    const int bundles = (a.S0 + a.S1 + 7) / 8 * 8;
    hipLaunchKernelGGL((conv_halo_wg_kernel<HWC, FI>), dim3((unsigned)(a.tiles * bundles)), dim3(HALO_NT), lds, st.stream,
                       a);
    if (!hip_ok(hipGetLastError(), "halo weight-gradient launch")) return 2;
    const long long total = (long long)d.Cout * d.Cin;
    // (64-filter tiles: one group of nine taps, every tap has S0 splits)
    // four outputs per thread from 128 x 128 filters on (same sums; in turns in one process 58.0 -> 56.3 us per call on
    // 256 -> 256 14x14 batch 128 channel-minor, 57.3 -> 56.5 channel-major, equal at batch 256); a 64 x 64 filter tensor
    // would be 144 workgroups that way (52.8 -> 54.6 us)
    // (in turns in one process: 278.9 -> 275.9 us per call on 512 -> 512 14x14 batch 256; from 1024 workgroups on)
    if (!HWC && total >= 1024 * 256 && total % 256 == 0 && (uintptr_t)dW % 16 == 0)
        hipLaunchKernelGGL(conv_halo_wg_reduce9_kernel, dim3((unsigned)(total / 256)), dim3(256), 0, st.stream, ws,
                           static_cast<half_t *>(dW), total, a.S0, a.S1, a.smax);
    else if (total >= 128 * 128)
        hipLaunchKernelGGL(conv_halo_wg_reduce4_kernel, dim3((unsigned)((total + 255) / 256), 9), dim3(256), 0, st.stream,
                           ws, static_cast<half_t *>(dW), total, a.S0, FI == 2 ? a.S0 : a.S1, a.smax, HWC ? d.Cin : 0);
    else
        hipLaunchKernelGGL(conv_halo_wg_reduce_kernel, dim3((unsigned)((total + 63) / 64), 9), dim3(256), 0, st.stream, ws,
                           static_cast<half_t *>(dW), total, a.S0, FI == 2 ? a.S0 : a.S1, a.smax, HWC ? d.Cin : 0);
    return hip_ok(hipGetLastError(), "halo weight-gradient reduce launch") ? 0 : 2;
}

// gb: the blocked, embedded gradient (top left of the grids at gb[cb * gstride + 0]; zero from the last padded
// position to conv_halo_wg_gradient_stride() positions); xb as for the forward kernel with conv_halo_wg_margin()
// readable chunks behind it; ws: conv_halo_wg_partial_bytes().
int conv_halo_wg_launch(const ConvTileDesc &d, const void *xb, const void *gb, long long gstride, float *ws, void *dW,
                        int Hp, int Wp, int S0, int S1) {
    const long long P = (long long)d.batch * Hp * Wp, Pd = conv_halo_wg_gradient_stride(d, Hp, Wp);
    HaloWgArgs a = {};
    a.xb = static_cast<const char *>(xb);
    a.gb = static_cast<const char *>(gb);
    a.ws = ws;
    a.Px = P;
    a.Pd = gstride;
    a.Cin = d.Cin; a.Cout = d.Cout; a.Wp = Wp;
    a.units = (int)(Pd / HWG_UNIT);
    a.tiles_ci = d.Cin / 64;
    a.tiles = (d.Cout / 128) * a.tiles_ci;
    a.S0 = S0; a.S1 = S1; a.smax = S0 > S1 ? S0 : S1;
    return halo_wg_run<false, 4>(a, d, ws, dW);
}

// Channel-minor 3x3 "same" layers (as conv_halo_hwc_fits) with whole 64-filter tiles and rows whose reach of two
// rows and two positions fits the 128 positions behind a unit; both tensors 16-byte aligned.
bool conv_halo_wg_hwc_fits(const ConvTileDesc &d, const void *X, const void *dY) {
    const int Wv = d.Win + 1;
    return d.in_hwc && d.KH == 3 && d.KW == 3 && d.sh == 1 && d.sw == 1 && d.padU == 1 && d.padD == 1 && d.padL == 1 &&
           d.padR == 1 && d.Ho == d.Hin && d.Wo == d.Win && d.Cin % 64 == 0 && d.Cout % 64 == 0 && 2 * Wv + 2 <= 128 &&
           reinterpret_cast<uintptr_t>(X) % 16 == 0 && reinterpret_cast<uintptr_t>(dY) % 16 == 0 &&
           (long long)(d.batch + 1) * (d.Hin + 1) * Wv + 2 * HWG_UNIT + 256 < ((long long)1 << 31);
}

// X: [batch][H][W][Cin], dY: [batch][H][W][Cout], dW: [Cout][3][3][Cin]; ws: conv_halo_wg_partial_bytes() of the
// virtual grid (Hp = H + 1, Wp = W + 1).
int conv_halo_wg_hwc_launch(const ConvTileDesc &d, const void *X, const void *dY, float *ws, void *dW, int S0, int S1) {
    State &st = state();
    const int Hp = d.Hin + 1, Wp = d.Win + 1;
    HaloWgArgs a = {};
    a.xb = static_cast<const char *>(X);
    a.gb = static_cast<const char *>(dY);
    a.zeros = static_cast<const char *>(st.zeros);
    if (!a.zeros) return 2;
    a.ws = ws;
    a.Cin = d.Cin; a.Cout = d.Cout; a.Wp = Wp; a.Hp = Hp; a.H = d.Hin; a.W = d.Win; a.batch = d.batch;
    a.units = (int)(conv_halo_wg_gradient_stride(d, Hp, Wp) / HWG_UNIT);
    a.tiles_ci = d.Cin / 64;
    const bool wide = d.Cout % 128 == 0;  // 128-filter tiles in two tap groups, else 64-filter tiles with all nine taps
    a.tiles = (d.Cout / (wide ? 128 : 64)) * a.tiles_ci;
    a.S0 = S0; a.S1 = wide ? S1 : 0; a.smax = S0 > a.S1 ? S0 : a.S1;
    magic31((unsigned)(Hp * Wp), &a.m_img, &a.s_img);
    magic31((unsigned)Wp, &a.m_row, &a.s_row);
    return wide ? halo_wg_run<true, 4>(a, d, ws, dW) : halo_wg_run<true, 2>(a, d, ws, dW);
}

}  // namespace ptl
