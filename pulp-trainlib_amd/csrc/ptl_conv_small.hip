// 3x3 fp16 convolution for small channel-major layers (up to 64 channels on either side, rows of whole 16-byte
// groups): forward, and input gradient as a forward pass with transposed, flipped filters.
//
// On such layers a call is a few microseconds of latency, not of work, so the kernel is one straight line per
// workgroup of sixteen waves (a single wave per SIMD issues an instruction every four or five cycles; four of them
// hide each other's issue gaps: 5.7 against 9.0 us for 16 -> 16 channels on 32x32 at batch 128), with nothing prepared
// by another launch:
//   * a workgroup owns R output rows of one sample and all filters.  Every thread issues all its global loads
//     at once: 16-byte pieces of the input rows (8 columns of one channel) and 16-byte pieces of the dense filter
//     tensor, both straight from the caller's tensors;
//   * the pieces are scattered into LDS as the MFMA operands want them: the input as [channel block][row][column]
//     chunks of 8 channels with the zero halo written in place (a wave's 64 lanes cover 8 channels x 8 rows, which
//     spreads the 2-byte writes over the banks), the filters as [filter][tap][channel];
//   * one barrier; then every wave takes jobs of 32 pixels x 32 filters: per tap and 16 channels one ds_read_b128
//     per operand (the pixel's chunk at position + tap offset) and one MFMA, filters as the MFMA rows and pixels as
//     the columns, so that the 32 lanes of a half-wave store 32 consecutive pixels of a filter.
#include "ptl_gemm_async.hpp"
#include "ptl_gemm_async.inc"
#include "ptl_conv_tile.hpp"
#include "ptl_structs.h"
#include "ptl_host.hpp"
#include "ptl_norm_fold.hpp"

namespace ptl {
namespace {

constexpr int CS_NT = 1024, CS_WAVES = CS_NT / 64;
constexpr int CS_ITEMS = 64;                      // wave-wide load items per workgroup, at most
constexpr int CS_IN_MAX = CS_ITEMS / CS_WAVES;  // input pieces per thread

struct ConvSmallArgs {
    const void *X, *Wt;
    void *Y;
    int Cin, Cout, Hin, Win, Ho, Wo, s, padU, padL;
    int dil;                // 2: the input is read zero-stuffed by two (tile rows and columns count the stuffed image)
    int R, tiles_per_img;   // output rows per workgroup
    int RR, TW, POS;        // input rows of a tile, padded row width, RR * TW
    int items;              // wave-wide load items: (channel block, column group, block of 64 / VEC rows)
    int halo_chunks, halo_w;  // zero chunks of a tile: channel blocks x rows x halo columns; halo columns per row
    unsigned magic_halo_w, magic_rr;
    int f_chunks, f_inner;  // 16-byte pieces of the filter tensor [outer][inner][9]; inner dimension
    int f_transposed;       // 0: outer = filter, inner = channel; 1: outer = channel, inner = filter, taps flipped
    int K;                  // filter extent both ways: 3, or 1 (one tap, kept in the first tap's place of a filter row)
    unsigned magic_inner9, magic_wo;
    int b_pitch, f_bytes;   // bytes per filter row in LDS, bytes of the filter tile
    int pgroups, mshift;    // jobs = groups of 32 pixels x (1 << mshift) blocks of 32 filters
    // Sums of the output (before it is rounded to T) and of its squares per filter, for a normalisation layer behind
    // the convolution:
    // stats[(filter * ntiles + tile) * 4 + {0, 1}]; NULL: not wanted.  stats_off: bytes into LDS of the jobs' sums.
    float *stats;
    int stats_off, ntiles;
    // Gradient epilogue (post != 0; input-gradient launches in front of a normalisation's backward pass): what is stored
    // is g = (T)(result [+ post_add]) [where post_mask > 0, else 0], and the sums are those of g and of g * post_x.
    // The three tensors have the shape of Y.
    const void *post_add, *post_mask, *post_x;
    int post, post_off;  // post_off: bytes into LDS of the waves' [32 filters][32 pixels] areas (see PostTile)
    // A normalisation in front of the layer, applied while the input is loaded (pre != 0; forward launches): X is the
    // normalisation's input, pre_part its sums ([channel][part][4], over pre_count elements per channel), and what the
    // taps see is out = [relu](norm(X) * weight + bias [+ pre_skip]), which the workgroup that owns a row also
    // writes to pre_out (every input row is owned by the tile whose output rows start at it).  pre_off: bytes into
    // LDS of the channels' {mean, weight / deviation, bias, -}.
    const float *pre_part;
    const void *pre_w, *pre_b, *pre_eps, *pre_skip;
    void *pre_out;
    float pre_count;
    int pre, pre_parts, pre_relu, pre_off;
    int ksplit, red_off;    // 1: the three filter rows of a job on three waves; bytes into LDS of their partial sums
    // per item: element offset into the sample (first channel, first tile row, column group), element offset into the
    // LDS tile, first tile row | first channel << 8 | column group << 16
    int item_g[CS_ITEMS], item_l[CS_ITEMS], item_rc[CS_ITEMS];
};

template <typename T>
union Piece {
    uint4 v;
    T e[16 / sizeof(T)];
};

// One halving step of a sum over the 16 lanes of a row: of the 2 * HALF values a lane holds it keeps the upper or the
// lower HALF (`up`) and adds the partner lane's copy of them, which arrives through the DPP pattern CTRL (a pattern that
// pairs lanes whose `up` differ).
template <int HALF, int CTRL>
__device__ inline void stats_fold(float (&s0)[16], float (&s1)[16], bool up) {
#pragma unroll
    for (int j = 0; j < HALF; ++j) {
        const float keep0 = up ? s0[j + HALF] : s0[j], send0 = up ? s0[j] : s0[j + HALF];
        const float keep1 = up ? s1[j + HALF] : s1[j], send1 = up ? s1[j] : s1[j + HALF];
        s0[j] = keep0 + __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(send0), CTRL, 0xF, 0xF, false));
        s1[j] = keep1 + __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(send1), CTRL, 0xF, 0xF, false));
    }
}

// T: element type; VEC = 16 / sizeof(T) elements make a 16-byte piece (8 halves, 4 floats): the channels of an LDS
// chunk, the columns of a global piece, the k values a lane hands to one MFMA step.
// Geometry of the gradient epilogue: a wave's LDS area holds a job's results as [32 filters][32 pixels + VEC] (the pad
// keeps the two filter groups a wave writes at once on different banks and the rows 16-byte aligned); a lane reads
// VEC pixels, LPR lanes share a filter, FPR filters make a round.
template <typename T>
struct PostTile {
    static constexpr int VEC = 16 / (int)sizeof(T), LPR = 32 / VEC, FPR = 64 / LPR, ROUNDS = 32 / FPR;
    static constexpr int PITCH = (32 + VEC) * (int)sizeof(T), BYTES = 32 * PITCH;
};
template <typename T>
struct PostIn {
    uint4 add[PostTile<T>::ROUNDS], mask[PostTile<T>::ROUNDS], x[PostTile<T>::ROUNDS];
};

template <typename T, int CINP, int F_MAX>
__device__ inline void conv_small_block(const ConvSmallArgs &a, int tile, char *smem) {
    constexpr int ES = (int)sizeof(T), VEC = 16 / ES, KSTEP = 2 * VEC;
    char *F = smem;
    T *Tl = reinterpret_cast<T *>(smem + a.f_bytes);  // [CINP / VEC][POS][VEC]
    const T *X = reinterpret_cast<const T *>(a.X);
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int b = tile / a.tiles_per_img, y0 = (tile - b * a.tiles_per_img) * a.R;
    const int iy0 = y0 * a.s - a.padU;

    // ---- the partial sums of a normalisation in front: asked for before anything else, added up behind the tile's loads
    constexpr int FOLD_R = CINP / 16;
    NormFoldRegs<FOLD_R> fold;
    if (a.pre) norm_fold_ask<FOLD_R>(fold, a.pre_part, a.pre_parts, 0, a.Cin, wave, lane);

    // ---- all global loads first
    Piece<T> xin[CS_IN_MAX];
    const int lrow = lane / VEC, lch = lane % VEC;
    const T *xs = X + ((size_t)b * a.Cin + lch) * a.Hin * a.Win + (iy0 + lrow) * a.Win;
#pragma unroll
    for (int k = 0; k < CS_IN_MAX; ++k) {
        const int item = wave + CS_WAVES * k;
        xin[k].v = make_uint4(0, 0, 0, 0);
        if (item < a.items) {
            const int rc = a.item_rc[item], rr = (rc & 255) + lrow, ch = ((rc >> 8) & 255) + lch, iy = iy0 + rr;
            if (a.dil == 2) {  // even rows of the stuffed image are rows of the tensor
                if (rr < a.RR && ch < a.Cin && iy >= 0 && !(iy & 1) && (iy >> 1) < a.Hin)
                    xin[k].v = *reinterpret_cast<const uint4 *>(
                        X + (((size_t)b * a.Cin + ch) * a.Hin + (iy >> 1)) * a.Win + VEC * (rc >> 16));
            } else if (rr < a.RR && ch < a.Cin && iy >= 0 && iy < a.Hin) {
                xin[k].v = *reinterpret_cast<const uint4 *>(xs + a.item_g[item]);
            }
        }
    }
    Piece<T> fin[F_MAX];
#pragma unroll
    for (int k = 0; k < F_MAX; ++k) {
        const int q = tid + CS_NT * k;
        if (q < a.f_chunks) fin[k].v = reinterpret_cast<const uint4 *>(a.Wt)[q];
    }
    if (a.pre) {  // the statistics of the normalisation in front: a wave per channel and round
        float4 *tab = reinterpret_cast<float4 *>(smem + a.pre_off);
        float2 sums[FOLD_R];
        norm_fold_take<FOLD_R>(fold, sums, a.pre_part, a.pre_parts, 0, a.Cin, wave, lane);
#pragma unroll
        for (int r = 0; r < FOLD_R; ++r) {
            const int c = wave + 16 * r;
            if (lane == 0 && c < a.Cin) {
                float mean, sd;
                norm_mean_sd(sums[r].x, sums[r].y, a.pre_count, (float)reinterpret_cast<const T *>(a.pre_eps)[0], mean, sd);
                tab[c] = make_float4(mean, (float)reinterpret_cast<const T *>(a.pre_w)[c] / sd,
                                     (float)reinterpret_cast<const T *>(a.pre_b)[c], 0.f);
            }
        }
    }

    // channels the tensor does not have must read as zeros on the filter side too (0 x garbage is not 0)
    if (a.Cin < CINP) {
        for (int i = tid; i < a.f_bytes / 16; i += CS_NT) reinterpret_cast<uint4 *>(F)[i] = make_uint4(0, 0, 0, 0);
        __syncthreads();
    }
    // ---- halo columns of the tile: whole chunks of zeros (a zero-stuffed input: the whole tile first)
    if (a.dil == 2) {
        for (int i = tid; i < (CINP / VEC) * a.POS; i += CS_NT) reinterpret_cast<uint4 *>(Tl)[i] = make_uint4(0, 0, 0, 0);
        __syncthreads();
    } else
    for (int i = tid; i < a.halo_chunks; i += CS_NT) {
        const int row = fast_div(i, a.magic_halo_w), hc = i - row * a.halo_w;  // row = channel block * RR + tile row
        const int cb = fast_div(row, a.magic_rr), rr = row - cb * a.RR;
        const int col = hc < a.padL ? hc : a.Win + hc;
        reinterpret_cast<uint4 *>(Tl)[cb * a.POS + rr * a.TW + col] = make_uint4(0, 0, 0, 0);
    }
    // ---- filter pieces -> [filter][tap][channel]: element (outer, inner, tap) of the dense tensor goes to
    // (filter, channel) = (outer, inner), or (inner, outer) with the taps flipped; the address moves with the indices
    if (a.K == 1) {  // [outer][inner]: element (outer, inner) goes to (filter, channel) or (channel, filter), tap place 0
#pragma unroll
        for (int k = 0; k < F_MAX; ++k) {
            const int q = tid + CS_NT * k;
            if (q < a.f_chunks) {
                const int e0 = q * VEC;
                int outer = fast_div(e0, a.magic_inner9), inner = e0 - outer * a.f_inner;
#pragma unroll
                for (int j = 0; j < VEC; ++j) {
                    const int m = a.f_transposed ? inner : outer, c = a.f_transposed ? outer : inner;
                    *reinterpret_cast<T *>(F + m * a.b_pitch + c * ES) = fin[k].e[j];
                    if (++inner == a.f_inner) {
                        inner = 0;
                        ++outer;
                    }
                }
            }
        }
    } else {
        const int step_tap = a.f_transposed ? -CINP * ES : CINP * ES;
        const int step_inner = (a.f_transposed ? a.b_pitch : ES) - 9 * step_tap;  // after the ninth tap step: tap 0, inner + 1
        const int step_outer = (a.f_transposed ? ES : a.b_pitch) - a.f_inner * (a.f_transposed ? a.b_pitch : ES);
#pragma unroll
        for (int k = 0; k < F_MAX; ++k) {
            const int q = tid + CS_NT * k;
            if (q < a.f_chunks) {
                const int e0 = q * VEC;
                const int outer = fast_div(e0, a.magic_inner9), rem = e0 - outer * a.f_inner * 9;
                const int inner = (rem * 7282) >> 16;  // rem / 9 for rem < 2^15
                const int tap = rem - inner * 9;
                const int m = a.f_transposed ? inner : outer, c = a.f_transposed ? outer : inner;
                const int at0 = m * a.b_pitch + ((a.f_transposed ? 8 - tap : tap) * CINP + c) * ES;
                // a piece is shorter than the nine taps of a filter plane, so it crosses into the next plane at most
                // once: its first n1 elements step through the taps from at0, the rest from the next plane's tap 0
                const int n1 = 9 - tap;
                const bool last = inner + 1 == a.f_inner;
                const int next0 = at0 + n1 * step_tap + step_inner + (last ? step_outer : 0);
                const int rest = next0 - n1 * step_tap;  // (element j >= n1 sits at rest + j * step_tap)
#pragma unroll
                for (int j = 0; j < VEC; ++j)
                    *reinterpret_cast<T *>(F + (j < n1 ? at0 : rest) + j * step_tap) = fin[k].e[j];
            }
        }
    }
    // (asked for only now, with the filter pieces out of their registers)
    Piece<T> skp[CS_IN_MAX];
    if (a.pre && a.pre_skip) {
        const T *ss = reinterpret_cast<const T *>(a.pre_skip) + (xs - X);
#pragma unroll
        for (int k = 0; k < CS_IN_MAX; ++k) {
            const int item = wave + CS_WAVES * k;
            skp[k].v = make_uint4(0, 0, 0, 0);
            if (item < a.items) {
                const int rc = a.item_rc[item], rr = (rc & 255) + lrow, ch = ((rc >> 8) & 255) + lch, iy = iy0 + rr;
                if (rr < a.RR && ch < a.Cin && iy >= 0 && iy < a.Hin)
                    skp[k].v = *reinterpret_cast<const uint4 *>(ss + a.item_g[item]);
            }
        }
    }
    // ---- input pieces -> [channel block][row][column] chunks
    T *tl = Tl + lrow * a.TW * VEC + lch;
    if (a.pre) __syncthreads();  // (the channels' statistics are in LDS)
#pragma unroll
    for (int k = 0; k < CS_IN_MAX; ++k) {
        const int item = wave + CS_WAVES * k;
        if (item < a.items && (a.item_rc[item] & 255) + lrow < a.RR) {
            if (a.pre) {
                const int rc = a.item_rc[item], ch = ((rc >> 8) & 255) + lch, iy = iy0 + (rc & 255) + lrow;
                if (ch < a.Cin && iy >= 0 && iy < a.Hin) {  // (a piece of the tensor, not of the padding)
                    const float4 t = reinterpret_cast<const float4 *>(smem + a.pre_off)[ch];
#pragma unroll
                    for (int j = 0; j < VEC; ++j) {
                        float v = norm_forward((float)xin[k].e[j], t.x, t.y, t.z);
                        if (a.pre_skip) v += (float)skp[k].e[j];
                        if (a.pre_relu) v = fmaxf(v, 0.f);
                        xin[k].e[j] = (T)v;
                    }
                    if (iy >= y0 * a.s && iy < (y0 + a.R) * a.s)
                        *reinterpret_cast<uint4 *>(reinterpret_cast<T *>(a.pre_out) + (xs - X) + a.item_g[item]) = xin[k].v;
                }
            }
            T *row = tl + a.item_l[item];
            const int step = VEC * a.dil;
#pragma unroll
            for (int j = 0; j < VEC; ++j) row[j * step] = xin[k].e[j];
        }
    }
    __syncthreads();

    // ---- jobs: 32 pixels x 32 filters
    const int kg = lane >> 5, lr = lane & 31;
    const int npix = min(a.R, a.Ho - y0) * a.Wo, jobs = a.pgroups << a.mshift;
    const uint4 *T4 = reinterpret_cast<const uint4 *>(Tl);
    const size_t plane = (size_t)a.Ho * a.Wo;
    // ---- the gradient epilogue (a.post: see ConvSmallArgs).  A job's 32 pixels are consecutive in memory (tiles are
    // whole rows), so its results, turned through a wave's own LDS area to [filter][pixel], meet the three tensors
    // in 16-byte pieces: a lane takes VEC pixels of one filter, PT::FPR filters a round.  The pieces of the tensors are
    // asked for before the job's MFMAs and used behind them.
    using PT = PostTile<T>;
    const int pf = lane / PT::LPR, pq = lane % PT::LPR;
    auto post_at = [&](int pg, int mb, int r, size_t &e) {
        const int f = mb * 32 + r * PT::FPR + pf, p = pg * 32 + pq * VEC;
        e = (((size_t)b * a.Cout + f) * a.Ho + y0) * a.Wo + p;
        return f < a.Cout && p < npix;  // (rows are whole pieces: a piece is inside the tile or outside)
    };
    auto post_load = [&](int pg, int mb, PostIn<T> &in) {
#pragma unroll
        for (int r = 0; r < PT::ROUNDS; ++r) {
            size_t e;
            const bool ok = post_at(pg, mb, r, e);
            in.add[r] = in.mask[r] = in.x[r] = make_uint4(0, 0, 0, 0);
            if (ok && a.post_add) in.add[r] = *reinterpret_cast<const uint4 *>(reinterpret_cast<const T *>(a.post_add) + e);
            if (ok && a.post_mask) in.mask[r] = *reinterpret_cast<const uint4 *>(reinterpret_cast<const T *>(a.post_mask) + e);
            if (ok) in.x[r] = *reinterpret_cast<const uint4 *>(reinterpret_cast<const T *>(a.post_x) + e);
        }
    };
    auto post_finish = [&](const f32x16 &acc, int job, int pg, int mb, const PostIn<T> &in) {
        char *area = smem + a.post_off + wave * PT::BYTES;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int f = 8 * (v >> 2) + (v & 3) + 4 * kg;
            *reinterpret_cast<T *>(area + f * PT::PITCH + lr * ES) = (T)acc[v];
        }
        // (the wave's lanes read what other lanes of it wrote: nothing to wait for but the order of the accesses)
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
        for (int r = 0; r < PT::ROUNDS; ++r) {
            size_t e;
            const bool ok = post_at(pg, mb, r, e);
            Piece<T> t, va, vm, vx;
            t.v = *reinterpret_cast<const uint4 *>(area + (r * PT::FPR + pf) * PT::PITCH + pq * 16);
            va.v = in.add[r];
            vm.v = in.mask[r];
            vx.v = in.x[r];
            float s0 = 0.f, s1 = 0.f;
#pragma unroll
            for (int j = 0; j < VEC; ++j) {
                T g = t.e[j];
                if (a.post_add) g = (T)((float)g + (float)va.e[j]);
                if (a.post_mask && !((float)vm.e[j] > 0.f)) g = (T)0;
                t.e[j] = g;
                s0 += (float)g;
                s1 += (float)g * (float)vx.e[j];
            }
            if (ok) *reinterpret_cast<uint4 *>(reinterpret_cast<T *>(a.Y) + e) = t.v;
            if (a.stats) {
                if (!ok) s0 = s1 = 0.f;  // (pixels beyond the tile's last one repeat it)
#pragma unroll
                for (int off = 1; off < PT::LPR; off <<= 1) {
                    s0 += __shfl_xor(s0, off);
                    s1 += __shfl_xor(s1, off);
                }
                if (pq == 0)
                    reinterpret_cast<float2 *>(smem + a.stats_off)[job * 32 + r * PT::FPR + pf] = make_float2(s0, s1);
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
    };
    // what a wave does with the finished sums of a job: store them, and add them up for the normalisation if asked
    auto finish = [&](const f32x16 &acc, int job, int pg, int mb, int py, int px) {
        if (a.post) {
            PostIn<T> in;
            post_load(pg, mb, in);
            post_finish(acc, job, pg, mb, in);
            return;
        }
        const int left = a.Cout - mb * 32 - 4 * kg;  // filters from this lane's first one
        const size_t at = (((size_t)b * a.Cout + mb * 32 + 4 * kg) * a.Ho + y0 + py) * a.Wo + px;
        if (pg * 32 + lr < npix) {
            T *out = reinterpret_cast<T *>(a.Y) + at;
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int f = 8 * (v >> 2) + (v & 3);
                if (f < left) out[f * plane] = (T)acc[v];
            }
        }
        if (a.stats) {
            // Sums over the job's 32 pixels of the results (and of their squares): a lane holds 16 filters of one
            // pixel.  Four exchanges inside a row of 16 lanes (mirrored row, mirrored half row, lanes 2 and 1 apart: DPP
            // moves, no LDS traffic) in each of which a lane keeps the half of its values that one bit of its lane
            // number selects and adds the partner's copy of them leave filter `lane % 16` summed over the row; the
            // two rows of a half-wave are added last.
            float s0[16], s1[16];
            // (lanes beyond the tile's last pixel repeat it and count as zeros; filters the layer does not have come
            // out as sums nobody reads)
            const bool pix_ok = pg * 32 + lr < npix;
#pragma unroll
            for (int v = 0; v < 16; ++v) s0[v] = pix_ok ? (float)(T)acc[v] : 0.f;  // the value as stored
#pragma unroll
            for (int v = 0; v < 16; ++v) s1[v] = s0[v] * s0[v];
            stats_fold<8, 0x140>(s0, s1, (lr & 8) != 0);
            stats_fold<4, 0x141>(s0, s1, (lr & 4) != 0);
            stats_fold<2, 0x4E>(s0, s1, (lr & 2) != 0);
            stats_fold<1, 0xB1>(s0, s1, (lr & 1) != 0);
            const float o0 = __shfl_xor(s0[0], 16), o1 = __shfl_xor(s1[0], 16);
            if (lr < 16) {
                const int f = 8 * (lr >> 2) + (lr & 3) + 4 * kg;  // value index lr of this lane's sixteen
                float2 *S = reinterpret_cast<float2 *>(smem + a.stats_off);
                S[job * 32 + f] = make_float2(s0[0] + o0, s1[0] + o1);
            }
        }
    };
    if (a.ksplit) {
        // A single sample: tiles of one or two jobs on many CUs, and the three filter rows of a job on three waves
        // (three SIMDs), whose sums meet in LDS.  A job's MFMAs keep one SIMD's matrix pipe busy for their whole
        // length - in fp32, at two k values per instruction, 4 us for 32 channels - so fewer jobs per CU and
        // a third of a job per SIMD is what shortens such a call (the split alone, with four jobs on a CU's four
        // SIMDs, changes nothing).  Larger batches keep the order of summation they have at every batch size.
        const int job = wave / 3, part = wave - 3 * job;
        const int pg = job >> a.mshift, mb = job - (pg << a.mshift);
        const bool active = job < jobs && pg * 32 < npix;
        f32x16 acc;
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[v] = 0.f;
        int py = 0, px = 0;
        if (active) {
            const int p = min(pg * 32 + lr, npix - 1);
            py = fast_div(p, a.magic_wo);
            px = p - py * a.Wo;
            const uint4 *prow = T4 + (py * a.TW + px) * a.s + kg * a.POS + part * a.TW;
            const char *frow = F + (mb * 32 + lr) * a.b_pitch + kg * 16 + part * 3 * CINP * ES;
#pragma unroll
            for (int ks = 0; ks < CINP / KSTEP; ++ks) {
                const uint4 *pr = prow + 2 * ks * a.POS;
#pragma unroll
                for (int kx = 0; kx < 3; ++kx)
                    mfma_step<T>(acc, *reinterpret_cast<const uint4 *>(frow + (kx * CINP + ks * KSTEP) * ES), pr[kx]);
            }
        }
        float *red = reinterpret_cast<float *>(smem + a.red_off);  // [job][filter row 1, 2][value][lane]
        if (active && part) {
#pragma unroll
            for (int v = 0; v < 16; ++v) red[((job * 2 + part - 1) * 16 + v) * 64 + lane] = acc[v];
        }
        __syncthreads();
        if (active && !part) {
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[v] += red[(job * 2 * 16 + v) * 64 + lane] + red[((job * 2 + 1) * 16 + v) * 64 + lane];
            finish(acc, job, pg, mb, py, px);
        }
    } else
    for (int job = wave; job < jobs; job += CS_NT / 64) {
        const int pg = job >> a.mshift, mb = job - (pg << a.mshift);
        if (pg * 32 >= npix) break;
        const int p = min(pg * 32 + lr, npix - 1);
        const int py = fast_div(p, a.magic_wo), px = p - py * a.Wo;
        const uint4 *prow = T4 + (py * a.TW + px) * a.s + kg * a.POS;
        const char *frow = F + (mb * 32 + lr) * a.b_pitch + kg * 16;
        PostIn<T> in;
        if (a.post) post_load(pg, mb, in);
        f32x16 acc;
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[v] = 0.f;
        if (a.K == 1) {
#pragma unroll
            for (int ks = 0; ks < CINP / KSTEP; ++ks)
                mfma_step<T>(acc, *reinterpret_cast<const uint4 *>(frow + ks * KSTEP * ES), prow[2 * ks * a.POS]);
        } else
#pragma unroll
        for (int ks = 0; ks < CINP / KSTEP; ++ks) {
            const uint4 *pk = prow + 2 * ks * a.POS;
#pragma unroll
            for (int ky = 0; ky < 3; ++ky) {
                const uint4 *pr = pk + ky * a.TW;
#pragma unroll
                for (int kx = 0; kx < 3; ++kx) {
                    const uint4 pf = pr[kx];
                    const uint4 ff = *reinterpret_cast<const uint4 *>(frow + ((ky * 3 + kx) * CINP + ks * KSTEP) * ES);
                    mfma_step<T>(acc, ff, pf);
                }
            }
        }
        if (a.post)
            post_finish(acc, job, pg, mb, in);
        else
            finish(acc, job, pg, mb, py, px);
    }
    if (a.stats) {  // the jobs' sums of a filter added in job order: one partial per workgroup and filter
        __syncthreads();
        if (tid < a.Cout) {
            const int mb = tid >> 5, f = tid & 31, npg = min(a.pgroups, (npix + 31) >> 5);
            const float2 *S = reinterpret_cast<const float2 *>(smem + a.stats_off);
            float t0 = 0.f, t1 = 0.f;
            for (int pg = 0; pg < npg; ++pg) {
                const float2 v = S[((pg << a.mshift) + mb) * 32 + f];
                t0 += v.x;
                t1 += v.y;
            }
            *reinterpret_cast<float2 *>(a.stats + ((size_t)tid * a.ntiles + tile) * 4) = make_float2(t0, t1);
        }
    }
}

// ---- Weight gradient of the same layers (unit stride, output rows as wide as input rows) -----------------------
// dW(co, ci, ky, kx) = sum over positions of dY(co, p) * X(ci, p + tap shift): the contraction runs over positions,
// which are contiguous in both channel-major tensors, so the MFMA operands (rows = filters, columns = channels,
// k = 8 consecutive output columns per lane half) are 16-byte pieces of the tensors as they lie in memory.  A lane per
// channel reading them from global memory keeps the address unit busy 64 cycles per load (one cache line per lane),
// so a workgroup first copies its tile - S samples x R output rows, every channel of the gradient and of the input
// with one row of halo above and below - into LDS with coalesced 16-byte loads, input rows separated by 8 zero
// elements (the left and right padding of neighbouring rows), rows outside the image as zeros.  Its waves are
// (filter row ky) x (32x32 block of the weight tensor) x (share of the positions); per k step a wave reads the
// gradient piece, the input piece and the input's two edge dwords, forms the three column taps by shifting whole
// elements in registers and issues three MFMAs.  The shares are added through LDS and the workgroup's partial sums go
// to ws[workgroup][block][tap][filter][channel] (filters and channels a tile really has); a second launch adds the workgroups and writes dW[co][ci][tap].
constexpr int WG_CHUNKS = 4;  // 16-byte pieces per thread and tensor, at most

struct WgSmallArgs {
    const void *X, *dY;
    float *ws;
    int batch, Cin, Cout, Hin, Win, Ho, Wo, padU, padL;
    int stride, rows_in;           // 1 or 2 (both ways); input rows a tile of R output rows meets: (R - 1) * stride + filter rows
    int nwg, S, R, tiles_per_img;  // workgroups; samples and output rows per tile (R = Ho when S > 1)
    int G, RG, Gin, R2G;           // 16-byte column groups per gradient row, per R of them; per input row, per rows_in of them
    int PY, PX, WP;                // LDS pitches in elements: gradient channel, input channel, input row
    int groups;                    // S * R * G
    int y_chunks, x_chunks, pad_chunks, pad_rows;  // pieces to copy; zero pieces (one per input row + one) and rows per channel
    unsigned magic_g, magic_gin, magic_rg, magic_r2g, magic_ychan, magic_xchan, magic_padrows, magic_tile, magic_cols;
    int cbi_n, combos, kparts;  // 32-channel blocks, (filter block, channel block) pairs, position shares
    int total;                  // Cout * Cin * taps
    int taps;                   // 9, or 1 for a 1x1 filter
    int bsplit, kparts_split;   // 1: a workgroup per (tile, block of the weight tensor); the position shares of such a workgroup
    int tiles;                  // tiles of samples and rows (= nwg, or nwg / combos with bsplit): the parts of the second launch
    int rows_kept, cols_kept, part_elems;  // filter rows and channels of a 32x32 tile that are stored; floats per workgroup in ws
};

// The two elements before and the two behind a 16-byte piece of a row: one dword of halves, two dwords of floats.
template <typename T>
struct EdgePair;
template <>
struct EdgePair<half_t> {
    typedef unsigned type;
};
template <>
struct EdgePair<float> {
    typedef uint2 type;
};

// elements D .. D + 3 of a row of floats of which c holds elements 0..3, p elements -2, -1 and n elements 4, 5
template <int D>
__device__ inline uint4 shifted_piece(const uint4 &c, const uint2 &p, const uint2 &n) {
    if constexpr (D == 0) return c;
    if constexpr (D == -1) return make_uint4(p.y, c.x, c.y, c.z);
    if constexpr (D == 1) return make_uint4(c.y, c.z, c.w, n.x);
    if constexpr (D == -2) return make_uint4(p.x, p.y, c.x, c.y);
    return make_uint4(c.z, c.w, n.x, n.y);
}

// elements D .. D + 7 of a row of halves of which c holds elements 0..7, p3 elements -2, -1 and n0 elements 8, 9
template <int D>
__device__ inline uint4 shifted_piece(const uint4 &c, unsigned p3, unsigned n0) {
    if constexpr (D == 0) return c;
    if constexpr (D == -1)
        return make_uint4(__builtin_amdgcn_alignbyte(c.x, p3, 2), __builtin_amdgcn_alignbyte(c.y, c.x, 2),
                          __builtin_amdgcn_alignbyte(c.z, c.y, 2), __builtin_amdgcn_alignbyte(c.w, c.z, 2));
    if constexpr (D == 1)
        return make_uint4(__builtin_amdgcn_alignbyte(c.y, c.x, 2), __builtin_amdgcn_alignbyte(c.z, c.y, 2),
                          __builtin_amdgcn_alignbyte(c.w, c.z, 2), __builtin_amdgcn_alignbyte(n0, c.w, 2));
    if constexpr (D == -2) return make_uint4(p3, c.x, c.y, c.z);
    return make_uint4(c.y, c.z, c.w, n0);
}

// STRIDE 2 (one column of left padding): an input row is kept as its even and its odd columns, each half behind a
// zero piece of its own - the eight input columns 2 x + kx - 1 that meet eight consecutive gradient columns x are
// then eight consecutive elements again: of the odd half one to the left (kx = 0), of the even half (1), of the odd
// half (2) - and gradient row y meets input rows 2 y + ky.
// K1: a 1x1 filter - one tap, no padding: every wave takes a share of the positions (no filter rows to split over).
template <typename T, int PADL, int STRIDE, bool K1 = false>
__device__ inline void wg_small_block(const WgSmallArgs &a, int wg, char *smem) {
    constexpr int VEC = 16 / (int)sizeof(T);
    typedef typename EdgePair<T>::type edge_t;
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // Layers of more than 32 channels on a side: a workgroup per 32 x 32 block of the weight tensor (bsplit) - it
    // copies the 32 gradient and the 32 input channels of its block only, splits the positions over all its waves
    // and leaves a quarter of the partial sums; `tile` is the tile of samples and rows it shares with its siblings.
    int tile = wg, co0 = 0, ci0 = 0, Cout = a.Cout, Cin = a.Cin, combos = a.combos, kparts = a.kparts, cbi_n = a.cbi_n;
    int part_elems = a.part_elems;
    if (a.bsplit) {
        tile = wg / a.combos;
        const int block = wg - tile * a.combos, bo = block / a.cbi_n;
        co0 = 32 * bo;
        ci0 = 32 * (block - bo * a.cbi_n);
        Cout = min(32, a.Cout - co0);
        Cin = min(32, a.Cin - ci0);
        combos = cbi_n = 1;
        kparts = a.kparts_split;
        part_elems = a.part_elems / a.combos;
    }
    const int y_chunks = Cout * a.groups, x_chunks = Cin * a.S * a.R2G, pad_chunks = Cin * a.pad_rows;
    T *Ys = reinterpret_cast<T *>(smem);
    T *Xs = Ys + Cout * a.PY;
    const T *gX = reinterpret_cast<const T *>(a.X), *gY = reinterpret_cast<const T *>(a.dY);
    // the tile: samples b0 .. b0 + S - 1, output rows y0 .. y0 + R - 1
    const int timg = tile / a.tiles_per_img;
    const int b0 = timg * a.S, y0 = (tile - timg * a.tiles_per_img) * a.R;

    // ---- copy: all loads first, then the LDS writes
    uint4 yv[WG_CHUNKS], xv[WG_CHUNKS];
    const int ychan = a.groups, xchan = a.S * a.R2G;  // pieces per channel
#pragma unroll
    for (int k = 0; k < WG_CHUNKS; ++k) {
        const int q = tid + CS_NT * k;
        yv[k] = xv[k] = make_uint4(0, 0, 0, 0);
        if (q < y_chunks) {
            const int co = fast_div(q, a.magic_ychan), rem = q - co * ychan;
            const int s = fast_div(rem, a.magic_rg), r2 = rem - s * a.RG;
            const int ly = fast_div(r2, a.magic_g), xg = r2 - ly * a.G;
            if (b0 + s < a.batch && y0 + ly < a.Ho)
                yv[k] = *reinterpret_cast<const uint4 *>(gY + (((size_t)(b0 + s) * a.Cout + co0 + co) * a.Ho + y0 + ly) * a.Wo + VEC * xg);
        }
        if (q < x_chunks) {
            const int ci = fast_div(q, a.magic_xchan), rem = q - ci * xchan;
            const int s = fast_div(rem, a.magic_r2g), r2 = rem - s * a.R2G;
            const int ly = fast_div(r2, a.magic_gin), xg = r2 - ly * a.Gin;
            const int iy = y0 * STRIDE - a.padU + ly;
            if (b0 + s < a.batch && iy >= 0 && iy < a.Hin)
                xv[k] = *reinterpret_cast<const uint4 *>(gX + (((size_t)(b0 + s) * a.Cin + ci0 + ci) * a.Hin + iy) * a.Win + VEC * xg);
        }
    }
    // zero pieces: in front of every input row and behind the last one; behind the last gradient group
    for (int q = tid; q < pad_chunks; q += CS_NT) {
        const int ci = fast_div(q, a.magic_padrows), j = q - ci * a.pad_rows;
        // (per row one piece, or one per half; the last one behind the last row)
        const int at = STRIDE == 1 ? j * a.WP : (j >> 1) * a.WP + (j & 1) * (VEC + a.Win / 2);
        *reinterpret_cast<uint4 *>(Xs + ci * a.PX + at) = make_uint4(0, 0, 0, 0);
    }
    for (int co = tid; co < Cout; co += CS_NT)
        *reinterpret_cast<uint4 *>(Ys + co * a.PY + a.groups * VEC) = make_uint4(0, 0, 0, 0);
#pragma unroll
    for (int k = 0; k < WG_CHUNKS; ++k) {
        const int q = tid + CS_NT * k;
        if (q < y_chunks) {
            const int co = fast_div(q, a.magic_ychan), rem = q - co * ychan;
            *reinterpret_cast<uint4 *>(Ys + co * a.PY + rem * VEC) = yv[k];
        }
        if (q < x_chunks) {
            const int ci = fast_div(q, a.magic_xchan), rem = q - ci * xchan;
            const int row = fast_div(rem, a.magic_gin), xg = rem - row * a.Gin;  // row = s * rows_in + ly
            T *at = Xs + ci * a.PX + row * a.WP + VEC;
            if constexpr (STRIDE == 1) {
                *reinterpret_cast<uint4 *>(at + VEC * xg) = xv[k];
            } else {
                const uint4 c = xv[k];
                uint2 even, odd;
                if constexpr (sizeof(T) == 2) {
                    even = make_uint2((c.x & 0xffffu) | (c.y << 16), (c.z & 0xffffu) | (c.w << 16));
                    odd = make_uint2((c.x >> 16) | (c.y & 0xffff0000u), (c.z >> 16) | (c.w & 0xffff0000u));
                } else {
                    even = make_uint2(c.x, c.z);
                    odd = make_uint2(c.y, c.w);
                }
                *reinterpret_cast<uint2 *>(at + (VEC / 2) * xg) = even;
                *reinterpret_cast<uint2 *>(at + VEC + a.Win / 2 + (VEC / 2) * xg) = odd;
            }
        }
    }
    __syncthreads();

    // ---- products
    const int ky = K1 ? 0 : wave % 3, rest = K1 ? wave : wave / 3;
    const int combo = rest % combos, kpart = rest / combos;
    const bool active = (K1 || wave < 15) && kpart < kparts;
    const int cbo = combo / cbi_n, cbi = combo - cbo * cbi_n;
    const int lr = lane & 31, kg = lane >> 5;
    const int nks = (a.groups + 1) >> 1;
    f32x16 acc[3];
#pragma unroll
    for (int kx = 0; kx < 3; ++kx)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[kx][v] = 0.f;
    if (active) {
        // filters and channels beyond the tensors repeat the last one (their rows and columns are never stored)
        const T *yrow = Ys + min(cbo * 32 + lr, Cout - 1) * a.PY;
        const T *xrow = Xs + min(cbi * 32 + lr, Cin - 1) * a.PX + ky * a.WP + VEC;
        constexpr int U = 4;  // k steps whose LDS reads are in flight together
        for (int ks0 = kpart; ks0 < nks; ks0 += U * kparts) {
            uint4 A[U], C[U], D[U];
            edge_t p3[U], n0[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                // (steps behind the last one read the zero piece of the gradient)
                const int gi = min(2 * (ks0 + u * kparts) + kg, a.groups);
                const int gx = min(gi, a.groups - 1);
                const int s = fast_div(gx, a.magic_rg), r2 = gx - s * a.RG;
                const int ly = fast_div(r2, a.magic_g), xg = r2 - ly * a.G;
                const T *xp = xrow + (s * a.rows_in + STRIDE * ly) * a.WP + VEC * xg;
                A[u] = *reinterpret_cast<const uint4 *>(yrow + gi * VEC);
                if constexpr (STRIDE == 1) {
                    C[u] = *reinterpret_cast<const uint4 *>(xp);
                    p3[u] = *reinterpret_cast<const edge_t *>(xp - 2);
                    n0[u] = *reinterpret_cast<const edge_t *>(xp + VEC);
                } else {  // C: the even half's piece; D, with the two elements before it: the odd half's
                    const T *xo = xp + VEC + a.Win / 2;
                    C[u] = *reinterpret_cast<const uint4 *>(xp);
                    D[u] = *reinterpret_cast<const uint4 *>(xo);
                    p3[u] = *reinterpret_cast<const edge_t *>(xo - 2);
                    n0[u] = p3[u];
                }
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                if constexpr (K1) {  // (the even half at stride 2: columns 2 x)
                    mfma_step<T>(acc[0], A[u], C[u]);
                } else if constexpr (STRIDE == 1) {
                    mfma_step<T>(acc[0], A[u], shifted_piece<0 - PADL>(C[u], p3[u], n0[u]));
                    mfma_step<T>(acc[1], A[u], shifted_piece<1 - PADL>(C[u], p3[u], n0[u]));
                    mfma_step<T>(acc[2], A[u], shifted_piece<2 - PADL>(C[u], p3[u], n0[u]));
                } else {
                    mfma_step<T>(acc[0], A[u], shifted_piece<-1>(D[u], p3[u], n0[u]));
                    mfma_step<T>(acc[1], A[u], C[u]);
                    mfma_step<T>(acc[2], A[u], D[u]);
                }
            }
        }
    }
    __syncthreads();  // the tiles are dead: the shares take their place
    // the shares of one (block, tap) side by side in LDS: [share][block][tap][32 filters][32 channels]
    float *L = reinterpret_cast<float *>(smem);
    if (active) {
#pragma unroll
        for (int kx = 0; kx < (K1 ? 1 : 3); ++kx) {
            float *t = L + ((kpart * combos + combo) * a.taps + ky * 3 + kx) * 1024 + lr;
#pragma unroll
            for (int v = 0; v < 16; ++v) t[(8 * (v >> 2) + 4 * kg + (v & 3)) * 32] = acc[kx][v];
        }
    }
    __syncthreads();
    // partial sums in tile order, [block][tap][filter row][channel] with the rows and channels the tensor has: thread t
    // (consecutive threads take consecutive elements of a tile: decoding an index of the weight tensor per element
    // would cost more than the sums, sixteen waves share the integer pipes); the second launch puts the sums where
    // the weight tensor wants them
    float *out = a.ws + (size_t)wg * part_elems;
    const int share = combos * a.taps * 1024, tile_elems = a.rows_kept * a.cols_kept;
    if (tile_elems == 1024) {  // whole tiles: thread t owns element t of every tile
        for (int t = 0; t < combos * a.taps; ++t) {
            const float *src = L + t * 1024 + tid;
            float sum = src[0];
            for (int kp = 1; kp < kparts; ++kp) sum += src[kp * share];
            out[t * 1024 + tid] = sum;
        }
        return;
    }
    for (int e = tid; e < part_elems; e += CS_NT) {
        const int t = fast_div(e, a.magic_tile), r = e - t * tile_elems;
        const int row = fast_div(r, a.magic_cols), col = r - row * a.cols_kept;
        const float *src = L + t * 1024 + row * 32 + col;
        float sum = src[0];
        for (int kp = 1; kp < kparts; ++kp) sum += src[kp * share];
        out[e] = sum;
    }
}

template <typename T>
__device__ inline void wg_small_any(const WgSmallArgs &a, int wg, char *smem) {
    if (a.taps == 1 && a.stride == 2)
        wg_small_block<T, 0, 2, true>(a, wg, smem);
    else if (a.taps == 1)
        wg_small_block<T, 0, 1, true>(a, wg, smem);
    else if (a.stride == 2)
        wg_small_block<T, 1, 2>(a, wg, smem);
    else if (a.padL == 1)
        wg_small_block<T, 1, 1>(a, wg, smem);
    else if (a.padL == 0)
        wg_small_block<T, 0, 1>(a, wg, smem);
    else
        wg_small_block<T, 2, 1>(a, wg, smem);
}

template <typename T>
__global__ __launch_bounds__(CS_NT) void wg_small_kernel(const WgSmallArgs a) {
    extern __shared__ __attribute__((aligned(16))) char smem[];
    wg_small_any<T>(a, blockIdx.x, smem);
}

template <typename T, int CINP, int F_MAX>
__global__ __launch_bounds__(CS_NT) void conv_small_kernel(const ConvSmallArgs a) {
    extern __shared__ __attribute__((aligned(16))) char smem[];
    conv_small_block<T, CINP, F_MAX>(a, blockIdx.x, smem);
}

// Weight gradient and input gradient of one layer in one launch: the first workgroups take the weight gradient's
// sample ranges (the longer jobs), the rest the input gradient's tiles.
template <typename T, int CINP, int F_MAX>
__global__ __launch_bounds__(CS_NT) void conv_small_bw_kernel(const ConvSmallArgs ig, const WgSmallArgs wg) {
    extern __shared__ __attribute__((aligned(16))) char smem[];
    if ((int)blockIdx.x < wg.nwg)
        wg_small_any<T>(wg, blockIdx.x, smem);
    else
        conv_small_block<T, CINP, F_MAX>(ig, blockIdx.x - wg.nwg, smem);
}

constexpr size_t WG_SMALL_LDS = 4 * 9 * 4096;  // shares x blocks <= 4 tiles of nine taps

template <typename T, int CINP, int F_MAX>
int launch_small(const ConvSmallArgs &a, int tiles, size_t lds, hipStream_t s, const WgSmallArgs *wg) {
    state().last_conv_resident = 2;
    static bool attr_set = false;
    if (!attr_set) {
        if (!hip_ok(hipFuncSetAttribute(reinterpret_cast<const void *>(conv_small_kernel<T, CINP, F_MAX>),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, 150 * 1024),
                    "hipFuncSetAttribute") ||
            !hip_ok(hipFuncSetAttribute(reinterpret_cast<const void *>(conv_small_bw_kernel<T, CINP, F_MAX>),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, 150 * 1024),
                    "hipFuncSetAttribute"))
            return 2;
        attr_set = true;
    }
    if (wg)
        hipLaunchKernelGGL((conv_small_bw_kernel<T, CINP, F_MAX>), dim3(tiles + wg->nwg), dim3(CS_NT),
                           lds > WG_SMALL_LDS ? lds : WG_SMALL_LDS, s, a, *wg);
    else
        hipLaunchKernelGGL((conv_small_kernel<T, CINP, F_MAX>), dim3(tiles), dim3(CS_NT), lds, s, a);
    return hip_ok(hipGetLastError(), "small convolution launch") ? 0 : 2;
}

// dW(co, ci, tap) = sum over workgroups of ws[workgroup][block][tap][filter row][channel]: 64 consecutive partial
// elements per workgroup of the reduction (coalesced reads), 16 groups of partials in parallel, eight loads in flight
// per thread; the few results are scattered to the weight tensor's order.
// PG groups of partials in parallel on 1024 / PG consecutive elements: 16 x 64 where a layer has many workgroups, 4 x 256
// up to 128 of them (a 64-channel layer has 32 and 36 864 elements: with 64 elements a block, 576 blocks of two loads a
// thread; at 128 workgroups the two forms are within half a per cent of each other in a ResNet-20 step's flush).
template <typename T, int PG>
__device__ inline void wg_small_reduce_part(const float *__restrict__ ws, T *__restrict__ dW, int block, int part_elems,
                                            int parts, int rows_kept, int cols_kept, int cbi_n, int Cout, int Cin,
                                            int taps) {
    constexpr int EPB = 1024 / PG;
    __shared__ float part_sum[PG][EPB];
    const int o = threadIdx.x % EPB, pg = threadIdx.x / EPB;
    const int i = block * EPB + o;
    float s = 0.f;
    if (i < part_elems) {
        const float *src = ws + i;
        int p = pg;
        for (; p + 7 * PG < parts; p += 8 * PG) {
            float v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = src[(size_t)(p + u * PG) * part_elems];
#pragma unroll
            for (int u = 0; u < 8; ++u) s += v[u];
        }
        float v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = p + u * PG < parts ? src[(size_t)(p + u * PG) * part_elems] : 0.f;
#pragma unroll
        for (int u = 0; u < 8; ++u) s += v[u];
    }
    part_sum[pg][o] = s;
    __syncthreads();
    if (pg == 0 && i < part_elems) {
#pragma unroll
        for (int q = 1; q < PG; ++q) s += part_sum[q][o];
        const int tile = i / (rows_kept * cols_kept), r = i - tile * rows_kept * cols_kept;
        const int combo = tile / taps, tap = tile - combo * taps;
        const int co = (combo / cbi_n) * 32 + r / cols_kept, ci = (combo % cbi_n) * 32 + r % cols_kept;
        if (co < Cout && ci < Cin) dW[(co * Cin + ci) * taps + tap] = (T)s;
    }
}

// (the shape of a layer decides its form, so that a deferred layer's sums have the bits of the immediate call's)
__host__ __device__ inline int wg_reduce_epb(int parts) { return parts <= 128 ? 256 : 64; }

template <typename T>
__device__ inline void wg_small_reduce_block(const float *__restrict__ ws, T *__restrict__ dW, int block, int part_elems,
                                             int parts, int rows_kept, int cols_kept, int cbi_n, int Cout, int Cin,
                                             int taps) {
    if (wg_reduce_epb(parts) == 256)
        wg_small_reduce_part<T, 4>(ws, dW, block, part_elems, parts, rows_kept, cols_kept, cbi_n, Cout, Cin, taps);
    else
        wg_small_reduce_part<T, 16>(ws, dW, block, part_elems, parts, rows_kept, cols_kept, cbi_n, Cout, Cin, taps);
}

template <typename T>
__global__ __launch_bounds__(1024) void wg_small_reduce_kernel(const float *__restrict__ ws, T *__restrict__ dW,
                                                               int part_elems, int parts, int rows_kept,
                                                               int cols_kept, int cbi_n, int Cout, int Cin, int taps) {
    wg_small_reduce_block<T>(ws, dW, blockIdx.x, part_elems, parts, rows_kept, cols_kept, cbi_n, Cout, Cin, taps);
}

// The same addition for the layers of a deferred batch in one launch: the blocks of all layers in one grid, a block
// finds its layer by the running block count.
struct WgFlushArgs {
    int count;
    int first_block[PTL_WG_BATCH_MAX + 1];
    const float *ws[PTL_WG_BATCH_MAX];
    void *grad[PTL_WG_BATCH_MAX];
    int shape[PTL_WG_BATCH_MAX][8];
};

template <typename T>
__global__ __launch_bounds__(1024) void wg_small_flush_kernel(const WgFlushArgs a) {
    int layer = 0;
    while (layer + 1 < a.count && (int)blockIdx.x >= a.first_block[layer + 1]) ++layer;
    const int *sh = a.shape[layer];
    wg_small_reduce_block<T>(a.ws[layer], reinterpret_cast<T *>(a.grad[layer]), (int)blockIdx.x - a.first_block[layer], sh[0],
                             sh[1], sh[2], sh[3], sh[4], sh[5], sh[6], sh[7]);
}

struct SmallPlan {
    ConvSmallArgs a;
    int tiles, cinp, per_thread;
    size_t lds;
};

// Fills the forward / input-gradient launch for `cu_budget` compute units; -1 when the layer does not fit.
template <typename T>
int plan_small(const ConvTileDesc &d, const void *X, const void *Wt, void *Y, int cu_budget, SmallPlan &p) {
    constexpr int ES = (int)sizeof(T), VEC = 16 / ES, RPI = 64 / VEC;  // element size, elements per piece, rows per item
    State &st = state();
    if (st.gemm_path != 0 && st.gemm_path != 6) return -1;  // (the other values select one of the other routes)
    const int K = d.KH;  // 3x3, or a single tap
    if (d.in_hwc || d.KH != d.KW || (K != 3 && K != 1) || d.sh != d.sw || d.sh < 1 || d.sh > 2) return -1;
    if (d.Cin > 64 || d.Cout > 64 || d.Win % VEC != 0 || d.x_sy != d.Win) return -1;
    if (d.x_sc != (long long)d.Hin * d.Win || d.x_sb != (long long)d.Cin * d.Hin * d.Win) return -1;
    if (d.padU < 0 || d.padU > 2 || d.padL < 0 || d.padL > 2 || d.padD < 0 || d.padR < 0 || d.padR > 8) return -1;
    if (reinterpret_cast<uintptr_t>(X) % 16 || reinterpret_cast<uintptr_t>(Wt) % 16) return -1;
    const long long f_elems = (long long)d.Cout * d.Cin * K * K;
    if (f_elems % VEC != 0) return -1;
    ConvSmallArgs &a = p.a;
    a = ConvSmallArgs();
    // dense filter tensor [outer][inner][3][3]: forward (filter, channel), or the input gradient's view of it
    if (d.w_base == 0 && d.w_sm == d.Cin * K * K && d.w_sc == K * K && d.w_sy == K && d.w_sx == 1) {
        a.f_transposed = 0;
        a.f_inner = d.Cin;
    } else if (d.w_base == K * K - 1 && d.w_sm == K * K && d.w_sc == d.Cout * K * K && d.w_sy == -K && d.w_sx == -1) {
        a.f_transposed = 1;
        a.f_inner = d.Cout;
    } else {
        return -1;
    }
    const int dil = d.in_dil == 2 ? 2 : 1;
    if (d.in_dil > 2 || (dil == 2 && d.sh != 1)) return -1;
    const int Hd = (d.Hin - 1) * dil + 1, Wd = (d.Win - 1) * dil + 1;  // the image the taps walk over
    const int s = d.sh, TW = Wd + d.padL + d.padR, THP = Hd + d.padU + d.padD;
    if ((d.Wo - 1) * s + K > TW || (d.Ho - 1) * s + K > THP || d.Wo >= 65536 || d.Ho * d.Wo >= 65536) return -1;
    const int cinp = d.Cin <= 16 ? 16 : d.Cin <= 32 ? 32 : 64, cblocks = cinp / VEC;
    const int mblocks = (d.Cout + 31) / 32;
    // rows per workgroup: the whole image, halved while that leaves the four waves a job each and the chip is not full
    int R = d.Ho;
    auto jobs_of = [&](int r) { return ((r * d.Wo + 31) / 32) * mblocks; };
    // (a single sample: down to one job per workgroup, whose three filter rows then go to three waves - see ksplit)
    const int min_jobs = d.batch == 1 && K == 3 ? 1 : 4;
    while ((long long)d.batch * ((d.Ho + R - 1) / R) < cu_budget && R % 2 == 0 && jobs_of(R / 2) >= min_jobs) R /= 2;
    auto items_of = [&](int r) { return cblocks * (d.Win / VEC) * ((((r - 1) * s + K) + RPI - 1) / RPI); };
    auto lds_of = [&](int r) { return (size_t)cblocks * ((r - 1) * s + K) * TW * 16; };
    const int pitch = K * K * cinp * ES + 16;  // (an odd multiple of 16 bytes)
    const size_t f_bytes = (size_t)mblocks * 32 * pitch;
    while (R > 1 && (items_of(R) > CS_ITEMS || f_bytes + lds_of(R) > 150 * 1024)) R = (R + 1) / 2;
    if (items_of(R) > CS_ITEMS || f_bytes + lds_of(R) > 150 * 1024) return -1;
    const long long tiles = (long long)d.batch * ((d.Ho + R - 1) / R);
    // beyond a few workgroups per CU the persistent kernels (filters loaded once per workgroup) are ahead where
    // both channel counts fill their 64-wide tiles; narrower layers stay ahead here for longer
    // (64 channels into 32 filters - the input gradient of a 32 -> 64 layer - has the resident-tile kernel's 32-filter
    // tile behind it in fp16 at unit stride)
    const bool persistent_next = d.Cin == 64 && (d.Cout == 64 || (d.Cout == 32 && ES == 2 && K == 3 && s == 1 && dil == 1));
    const long long tile_limit = (persistent_next ? 4LL : 16LL) * st.num_cu;
    if (st.gemm_path != 6 && tiles > tile_limit) return -1;
    if (tiles >= (1LL << 31) / 256) return -1;
    a.X = X;
    a.Wt = Wt;
    a.Y = Y;
    a.Cin = d.Cin; a.Cout = d.Cout; a.Hin = d.Hin; a.Win = d.Win; a.Ho = d.Ho; a.Wo = d.Wo;
    a.s = s; a.padU = d.padU; a.padL = d.padL;
    a.dil = dil;
    a.R = R; a.tiles_per_img = (d.Ho + R - 1) / R;
    a.RR = (R - 1) * s + K; a.TW = TW; a.POS = a.RR * TW;
    a.K = K;
    const int G = d.Win / VEC, RRB = (a.RR + RPI - 1) / RPI;
    a.items = cblocks * G * RRB;
    for (int item = 0; item < a.items; ++item) {
        const int rblk = item % RRB, t = item / RRB, g = t % G, cb = t / G;
        a.item_g[item] = (cb * VEC * d.Hin + rblk * RPI) * d.Win + VEC * g;
        a.item_l[item] = ((cb * a.POS + rblk * RPI * TW) + d.padL + dil * VEC * g) * VEC;
        a.item_rc[item] = (rblk * RPI) | ((cb * VEC) << 8) | (g << 16);
    }
    if (a.RR + RPI > 255) return -1;  // (rows are 8 bits of item_rc)
    a.halo_w = dil == 2 ? 1 : TW - d.Win;  // (a zero-stuffed input zeroes its whole tile instead)
    a.halo_chunks = cblocks * a.RR * a.halo_w;
    a.magic_halo_w = magic_of(a.halo_w);
    a.magic_rr = magic_of(a.RR);
    a.f_chunks = (int)(f_elems / VEC);
    a.magic_inner9 = magic_of(a.f_inner * K * K);
    a.magic_wo = magic_of(d.Wo);
    a.b_pitch = pitch; a.f_bytes = (int)f_bytes;
    a.pgroups = (R * d.Wo + 31) / 32; a.mshift = mblocks - 1;
    if (f_elems >= 65536 || a.f_inner * 9 >= 65536) return -1;  // (quotients by reciprocal multiplication)
    if (a.halo_chunks >= 65536 || a.RR * cblocks >= 65536) return -1;
    p.tiles = (int)tiles;
    p.lds = f_bytes + lds_of(R);
    // a single sample: the filter rows of a job on separate waves, 8 KB of partial sums per job behind the tile
    const int jobs = a.pgroups << a.mshift;
    if (d.batch == 1 && K == 3 && 3 * jobs <= CS_WAVES && (p.lds + 15) / 16 * 16 + (size_t)jobs * 2 * 16 * 64 * sizeof(float) <= 150 * 1024) {
        a.ksplit = 1;
        a.red_off = (int)((p.lds + 15) / 16 * 16);
        p.lds = a.red_off + (size_t)jobs * 2 * 16 * 64 * sizeof(float);
    }
    p.cinp = cinp;
    p.per_thread = (a.f_chunks + CS_NT - 1) / CS_NT;
    if (p.per_thread > (cinp == 16 ? 2 : cinp == 32 ? 3 : 5)) return -1;
    return 0;
}

template <typename T>
int dispatch_small(const SmallPlan &p, const WgSmallArgs *wg) {
    hipStream_t s = state().stream;
    if (p.cinp == 16)
        return p.per_thread <= 1 ? launch_small<T, 16, 1>(p.a, p.tiles, p.lds, s, wg) : launch_small<T, 16, 2>(p.a, p.tiles, p.lds, s, wg);
    if (p.cinp == 32)
        return p.per_thread <= 2 ? launch_small<T, 32, 2>(p.a, p.tiles, p.lds, s, wg) : launch_small<T, 32, 3>(p.a, p.tiles, p.lds, s, wg);
    return p.per_thread <= 3 ? launch_small<T, 64, 3>(p.a, p.tiles, p.lds, s, wg) : launch_small<T, 64, 5>(p.a, p.tiles, p.lds, s, wg);
}

// Fills the weight-gradient launch of the forward layer `d` (partial sums in the workspace); -1 when it does not fit.
template <typename T>
int plan_wg(const ConvTileDesc &d, const void *X, const void *dY, int max_wg, bool alone, WgSmallArgs &w) {
    constexpr int ES = (int)sizeof(T), VEC = 16 / ES;
    State &st = state();
    if (st.gemm_path != 0 && st.gemm_path != 6) return -1;  // (the other values select one of the other routes)
    const int K = d.KH;  // 3x3, or a single tap
    if (d.in_hwc || d.KH != d.KW || (K != 3 && K != 1) || d.sh != d.sw || d.sh < 1 || d.sh > 2) return -1;
    const int st2 = d.sh == 2;
    if (d.Cin > 64 || d.Cout > 64 || d.Win % VEC != 0 || d.Wo % VEC != 0 || d.x_sy != d.Win) return -1;
    if (d.x_sc != (long long)d.Hin * d.Win || d.x_sb != (long long)d.Cin * d.Hin * d.Win) return -1;
    if (d.padU < 0 || d.padL < 0 || d.padL > 2) return -1;
    // unit stride: a gradient row as long as an input row; stride 2: half as long, one column of left padding, and
    // the input columns the last gradient column meets inside the row
    if (!st2 && d.Wo != d.Win) return -1;
    if (st2 && (d.padL != (K == 3 ? 1 : 0) || d.Win % (2 * VEC) != 0 || d.Wo * 2 != d.Win)) return -1;
    if (K == 1 && d.padL != 0) return -1;
    if (reinterpret_cast<uintptr_t>(X) % 16 || reinterpret_cast<uintptr_t>(dY) % 16) return -1;
    w = WgSmallArgs();
    w.taps = K * K;
    w.total = d.Cout * d.Cin * w.taps;
    if (w.total >= 65536) return -1;
    const long long positions = (long long)d.batch * d.Ho * d.Wo;
    // large calls keep the tiled weight-gradient kernels, and so do small calls for the weight gradient alone (measured
    // 12.0 against 13.7 us for 32 -> 32 on 16x16 at batch 128, 16.7 against 20.0 us for 64 -> 64 on 8x8, but 8.8
    // against 8.4 us for 16 -> 32 on 32x32 at one sample: below a few thousand positions what this kernel buys is
    // the input gradient riding along in the same launch)
    if (st.gemm_path != 6 && (positions > 262144 || (alone && positions < 8192))) return -1;
    // (a single tap alone: beyond 65536 positions the streaming GEMM with its k split is ahead - 10.0 against 13.6 us
    // for 32 -> 32 on 16x16 at batch 512)
    if (st.gemm_path != 6 && K == 1 && alone && positions > 65536) return -1;
    w.G = d.Wo / VEC;
    w.Gin = d.Win / VEC;
    w.stride = d.sh;
    w.WP = d.Win + (st2 ? 2 : 1) * VEC;
    auto rows_in = [&](int R) { return (R - 1) * d.sh + K; };
    // pitches of 16 bytes mod 128: consecutive channels 16 bytes apart in the banks
    auto round_pitch = [](int n) { return n + ((VEC - n % (8 * VEC)) + 8 * VEC) % (8 * VEC); };
    // more than one 32 x 32 block of the weight tensor: a workgroup per block (32 channels of either tensor in LDS,
    // every wave on a share of the positions, a block's worth of partial sums to write)
    const int blocks = ((d.Cin + 31) / 32) * ((d.Cout + 31) / 32);
    w.bsplit = blocks > 1;
    const int co_wg = w.bsplit ? 32 : d.Cout, ci_wg = w.bsplit ? 32 : d.Cin;  // channels a workgroup copies, at most
    auto lds_of = [&](int S, int R) {
        const int py = round_pitch(S * R * d.Wo + VEC), px = round_pitch((S * rows_in(R) + 1) * w.WP);
        return ((size_t)co_wg * py + (size_t)ci_wg * px) * ES;
    };
    auto chunks_ok = [&](int S, int R) {
        return (long long)co_wg * S * R * w.G <= WG_CHUNKS * CS_NT && (long long)ci_wg * S * rows_in(R) * w.Gin <= WG_CHUNKS * CS_NT &&
               lds_of(S, R) <= WG_SMALL_LDS;
    };
    // tiles: whole samples while the partial sums stay within about 5 MB (S samples each otherwise), rows of a
    // sample split while that fills more of `max_wg` workgroups and leaves the waves eight k steps each
    int S = 1, R = d.Ho;
    const long long part_bytes = (long long)((d.Cin + 31) / 32) * ((d.Cout + 31) / 32) * w.taps * (d.Cout < 32 ? d.Cout : 32) * (d.Cin < 32 ? d.Cin : 32) * 4;
    while ((long long)((d.batch + S - 1) / S) * part_bytes > (5LL << 20) && chunks_ok(S * 2, R)) S *= 2;
    if (S == 1)
        while (R % 2 == 0 && (long long)d.batch * (d.Ho / R) * 2 * blocks <= max_wg && (R / 2) * w.G >= 16 &&
               (long long)d.batch * (d.Ho / R) * 2 * part_bytes <= (5LL << 20))
            R /= 2;
    while (!chunks_ok(S, R) && R % 2 == 0 && S == 1) R /= 2;
    if (!chunks_ok(S, R)) return -1;
    w.S = S; w.R = R;
    w.tiles_per_img = (d.Ho + R - 1) / R;
    w.tiles = ((d.batch + S - 1) / S) * w.tiles_per_img;
    w.nwg = w.tiles * (w.bsplit ? blocks : 1);
    w.rows_in = rows_in(R);
    w.RG = R * w.G; w.R2G = w.rows_in * w.Gin;
    w.groups = S * w.RG;
    w.PY = round_pitch(w.groups * VEC + VEC);
    w.pad_rows = (st2 ? 2 : 1) * S * w.rows_in + 1;
    w.PX = round_pitch((S * w.rows_in + 1) * w.WP);
    w.y_chunks = co_wg * w.groups;
    w.x_chunks = ci_wg * S * w.R2G;
    w.pad_chunks = ci_wg * w.pad_rows;
    if (w.y_chunks >= 65536 || w.x_chunks >= 65536 || w.pad_chunks >= 65536) return -1;  // (reciprocal multiplication)
    w.magic_g = magic_of(w.G);
    w.magic_gin = magic_of(w.Gin);
    w.magic_rg = magic_of(w.RG);
    w.magic_r2g = magic_of(w.R2G);
    w.magic_ychan = magic_of(w.groups);
    w.magic_xchan = magic_of(S * w.R2G);
    w.magic_padrows = magic_of(w.pad_rows);
    w.cbi_n = (d.Cin + 31) / 32;
    w.combos = w.cbi_n * ((d.Cout + 31) / 32);
    w.kparts = (K == 1 ? 16 : 4) / w.combos;
    w.kparts_split = K == 1 ? 16 : 4;
    w.rows_kept = d.Cout < 32 ? d.Cout : 32;
    w.cols_kept = d.Cin < 32 ? d.Cin : 32;
    w.part_elems = w.combos * w.taps * w.rows_kept * w.cols_kept;
    w.magic_tile = magic_of(w.rows_kept * w.cols_kept);
    w.magic_cols = magic_of(w.cols_kept);
    w.X = X;
    w.dY = dY;
    w.batch = d.batch; w.Cin = d.Cin; w.Cout = d.Cout; w.Hin = d.Hin; w.Win = d.Win; w.Ho = d.Ho; w.Wo = d.Wo;
    w.padU = d.padU; w.padL = d.padL;
    w.ws = workspace((size_t)w.tiles * w.part_elems * sizeof(float));
    return w.ws ? 0 : 2;
}

template <typename T>
int reduce_wg(const WgSmallArgs &w, void *dW) {
    hipLaunchKernelGGL(wg_small_reduce_kernel<T>, dim3((w.part_elems + wg_reduce_epb(w.tiles) - 1) / wg_reduce_epb(w.tiles)), dim3(1024), 0,
                       state().stream, w.ws,
                       reinterpret_cast<T *>(dW), w.part_elems, w.tiles, w.rows_kept, w.cols_kept, w.cbi_n, w.Cout, w.Cin, w.taps);
    return hip_ok(hipGetLastError(), "small weight gradient reduction launch") ? 0 : 2;
}

}  // namespace

static ::ptl_norm_stats *g_norm_stats = nullptr;  // where the forward pass leaves the sums of its output, if anywhere

void conv_small_stats_to(::ptl_norm_stats *st) { g_norm_stats = st; }

static const ConvPreNorm *g_pre_norm = nullptr;  // the normalisation the next forward call applies, if any
static bool g_pre_taken = false;

void conv_small_pre_to(const ConvPreNorm *pre) {
    g_pre_norm = pre;
    g_pre_taken = false;
}
bool conv_small_pre_pending() { return g_pre_norm && !g_pre_taken; }

template <typename T>
int conv_small(const ConvTileDesc &d, const void *X, const void *Wt, void *Y) {
    SmallPlan p;
    const ConvPreNorm *pre = g_pre_norm;
    if (int rc = plan_small<T>(d, X, Wt, Y, state().num_cu, p)) return pre ? CONV_PRE_REFUSED : rc;
    if (pre) {
        // the table of the channels' statistics behind the tile; every input row must be a row that some tile both
        // loads and owns (rows [y0 * s, (y0 + R) * s) of the tile at output row y0)
        auto aligned = [](const void *q) { return reinterpret_cast<uintptr_t>(q) % 16 == 0; };
        const size_t off = (p.lds + 15) / 16 * 16, need = (size_t)d.Cin * sizeof(float4);
        const bool ok = X == pre->out && pre->x && pre->weight && pre->bias && pre->eps && pre->part && pre->parts > 0 &&
                        aligned(pre->x) && aligned(pre->out) && aligned(pre->skip) && aligned(pre->part) &&
                        p.a.dil == 1 && d.padU <= d.KH - d.sh && (long long)d.Ho * d.sh >= d.Hin &&
                        pre->count == (size_t)d.batch * d.Hin * d.Win && off + need <= 150 * 1024;
        if (!ok) return CONV_PRE_REFUSED;
        p.a.X = pre->x;
        p.a.pre = 1;
        p.a.pre_out = pre->out;
        p.a.pre_skip = pre->skip;
        p.a.pre_w = pre->weight;
        p.a.pre_b = pre->bias;
        p.a.pre_eps = pre->eps;
        p.a.pre_part = pre->part;
        p.a.pre_parts = pre->parts;
        p.a.pre_relu = pre->relu;
        p.a.pre_count = (float)d.batch * (float)(d.Hin * d.Win);
        p.a.pre_off = (int)off;
        p.lds = off + need;
        g_pre_taken = true;
    }
    if (::ptl_norm_stats *st = g_norm_stats) {
        // a pair of sums per job (32 pixels x 32 filters) in LDS behind the tile, a partial per workgroup and filter
        // in the caller's buffer; a layer whose jobs or partials do not fit goes without
        const size_t off = (p.lds + 15) / 16 * 16, need = (size_t)(p.a.pgroups << p.a.mshift) * 32 * sizeof(float2);
        const size_t part_bytes = (size_t)d.Cout * p.tiles * 4 * sizeof(float);
        if (off + need <= 150 * 1024 && st->part && part_bytes <= st->bytes &&
            reinterpret_cast<uintptr_t>(st->part) % 16 == 0) {
            p.a.stats = st->part;
            p.a.stats_off = (int)off;
            p.a.ntiles = p.tiles;
            p.lds = off + need;
            st->parts = p.tiles;
            st->channels = d.Cout;
            st->count = (size_t)d.batch * d.Ho * d.Wo;
            st->valid = 1;
        }
    }
    const int rc = dispatch_small<T>(p, nullptr);
    if (pre && rc == 0) state().last_conv_resident = 3;
    return rc;
}

static ::ptl_wg_batch *g_wg_defer = nullptr;  // where a backward call leaves its partial sums, if anywhere

void conv_small_defer_to(::ptl_wg_batch *batch) { g_wg_defer = batch; }

// A deferred layer: its partial sums go to the batch's buffer (if they fit) and wait for the flush (not when dW is a
// staging copy of a host tensor: the call copies it back when it returns).  Returns the batch, or null.
static ::ptl_wg_batch *defer_slot(WgSmallArgs &w, bool may_defer, size_t &need) {
    ::ptl_wg_batch *b = may_defer ? g_wg_defer : nullptr;
    need = ((size_t)w.tiles * w.part_elems * sizeof(float) + 255) / 256 * 256;
    const bool defer = b && b->buf && b->count >= 0 && b->count < PTL_WG_BATCH_MAX && b->used % 256 == 0 &&
                       b->used <= b->bytes && need <= b->bytes - b->used && reinterpret_cast<uintptr_t>(b->buf) % 256 == 0;
    if (!defer) return nullptr;
    w.ws = reinterpret_cast<float *>(static_cast<char *>(b->buf) + b->used);
    return b;
}
static void defer_record(::ptl_wg_batch *b, const WgSmallArgs &w, void *dW, size_t need) {
    const int at = b->count++;
    b->offset[at] = b->used;
    b->grad[at] = dW;
    const int shape[8] = {w.part_elems, w.tiles, w.rows_kept, w.cols_kept, w.cbi_n, w.Cout, w.Cin, w.taps};
    for (int i = 0; i < 8; ++i) b->shape[8 * at + i] = shape[i];
    b->used += need;
}

float *wg_batch_reserve(::ptl_wg_batch *b, void *dW, int parts, int filters, int channels, int taps) {
    if (!b || !dW || parts <= 0 || filters <= 0 || filters > 32 || channels <= 0 || taps <= 0) return nullptr;
    // (one block of filters, the channels in blocks of 32: what the flush's index arithmetic covers)
    WgSmallArgs w = WgSmallArgs();
    w.cbi_n = (channels + 31) / 32;
    w.rows_kept = filters;
    w.cols_kept = channels < 32 ? channels : 32;
    w.part_elems = w.cbi_n * taps * w.rows_kept * w.cols_kept;
    w.tiles = parts;
    w.Cout = filters;
    w.Cin = channels;
    w.taps = taps;
    ::ptl_wg_batch *saved = g_wg_defer;
    g_wg_defer = b;
    size_t need;
    ::ptl_wg_batch *slot = defer_slot(w, true, need);
    g_wg_defer = saved;
    if (!slot) return nullptr;
    defer_record(slot, w, dW, need);
    return w.ws;
}

template <typename T>
int conv_small_wg(const ConvTileDesc &d, const void *X, const void *dY, void *dW, bool may_defer) {
    WgSmallArgs w;
    if (int rc = plan_wg<T>(d, X, dY, state().num_cu, true, w)) return rc;
    size_t need;
    ::ptl_wg_batch *b = defer_slot(w, may_defer, need);
    static bool attr_set = false;
    if (!attr_set) {
        if (!hip_ok(hipFuncSetAttribute(reinterpret_cast<const void *>(wg_small_kernel<T>),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, 150 * 1024),
                    "hipFuncSetAttribute"))
            return 2;
        attr_set = true;
    }
    state().last_conv_resident = 2;
    hipLaunchKernelGGL(wg_small_kernel<T>, dim3(w.nwg), dim3(CS_NT), WG_SMALL_LDS, state().stream, w);
    if (!hip_ok(hipGetLastError(), "small weight gradient launch")) return 2;
    if (!b) return reduce_wg<T>(w, dW);
    defer_record(b, w, dW, need);
    return 0;
}


// What the input gradient of the one-call backward does in its epilogue, and where its sums go, if anything
static const ::ptl_grad_post *g_grad_post = nullptr;
static ::ptl_norm_stats *g_grad_sums = nullptr;

void conv_small_post_to(const ::ptl_grad_post *post, ::ptl_norm_stats *sums) {
    g_grad_post = post;
    g_grad_sums = sums;
}

template <typename T>
int conv_small_bw(const ConvTileDesc &fwd, const ConvTileDesc &ig, const void *X, const void *dY, const void *Wt,
                  void *dW, void *dX, bool may_defer) {
    WgSmallArgs w;
    if (int rc = plan_wg<T>(fwd, X, dY, state().num_cu / 2, false, w)) return rc;
    SmallPlan p;
    const int budget = state().num_cu - w.nwg;
    if (int rc = plan_small<T>(ig, dY, Wt, dX, budget > 32 ? budget : 32, p)) return rc;
    size_t need;
    ::ptl_wg_batch *b = defer_slot(w, may_defer, need);
    if (g_grad_post && g_grad_sums && may_defer && g_grad_post->x) {
        // the gradient epilogue: the jobs' sums in LDS behind the tile, a partial per workgroup and channel in the caller's
        // buffer - like the forward sums; a layer whose jobs or partials do not fit goes without (sums->valid stays 0)
        ::ptl_norm_stats *st = g_grad_sums;
        const size_t off = (p.lds + 15) / 16 * 16, need_lds = (size_t)(p.a.pgroups << p.a.mshift) * 32 * sizeof(float2);
        const size_t part_bytes = (size_t)ig.Cout * p.tiles * 4 * sizeof(float);
        const size_t off2 = (off + need_lds + 15) / 16 * 16, need2 = (size_t)CS_WAVES * PostTile<T>::BYTES;
        auto aligned = [](const void *q) { return reinterpret_cast<uintptr_t>(q) % 16 == 0; };
        if (off2 + need2 <= 150 * 1024 && st->part && part_bytes <= st->bytes && aligned(st->part) && aligned(dX) &&
            aligned(g_grad_post->add) && aligned(g_grad_post->mask) && aligned(g_grad_post->x) &&
            ig.Wo % PostTile<T>::VEC == 0) {
            p.a.post = 1;
            p.a.post_off = (int)off2;
            p.a.post_add = g_grad_post->add;
            p.a.post_mask = g_grad_post->mask;
            p.a.post_x = g_grad_post->x;
            p.a.stats = st->part;
            p.a.stats_off = (int)off;
            p.a.ntiles = p.tiles;
            p.lds = off2 + need2;
            st->parts = p.tiles;
            st->channels = ig.Cout;
            st->count = (size_t)ig.batch * ig.Ho * ig.Wo;
            st->valid = 1;
        }
    }
    if (int rc = dispatch_small<T>(p, &w)) {
        if (g_grad_sums) g_grad_sums->valid = 0;
        return rc;
    }
    if (!b) return reduce_wg<T>(w, dW);
    defer_record(b, w, dW, need);
    return 0;
}

template <typename T>
int conv_small_flush(::ptl_wg_batch *b) {
    if (!b || b->count < 0 || b->count > PTL_WG_BATCH_MAX || (b->count > 0 && !b->buf)) {
        set_error("weight-gradient flush: invalid batch");
        return 1;
    }
    if (b->count == 0) {
        b->used = 0;
        return 0;
    }
    if (!ensure_init()) return 2;
    WgFlushArgs a;
    a.count = b->count;
    int blocks = 0;
    for (int i = 0; i < b->count; ++i) {
        const int *shape = b->shape + 8 * i;
        if (b->offset[i] % 4 || b->offset[i] > b->bytes || !b->grad[i] || shape[0] <= 0 || shape[1] <= 0 || shape[2] <= 0 ||
            shape[3] <= 0 || shape[4] <= 0 || shape[7] <= 0 ||
            (size_t)shape[0] * shape[1] * sizeof(float) > b->bytes - b->offset[i]) {
            set_error("weight-gradient flush: layer %d of the batch does not describe partial sums inside its buffer", i);
            return 1;
        }
        a.first_block[i] = blocks;
        blocks += (shape[0] + wg_reduce_epb(shape[1]) - 1) / wg_reduce_epb(shape[1]);
        a.ws[i] = reinterpret_cast<const float *>(static_cast<const char *>(b->buf) + b->offset[i]);
        a.grad[i] = b->grad[i];
        for (int k = 0; k < 8; ++k) a.shape[i][k] = shape[k];
    }
    a.first_block[b->count] = blocks;
    hipLaunchKernelGGL(wg_small_flush_kernel<T>, dim3(blocks), dim3(1024), 0, state().stream, a);
    b->count = 0;
    b->used = 0;
    return hip_ok(hipGetLastError(), "weight-gradient flush launch") ? 0 : 2;
}

template int conv_small_flush<half_t>(::ptl_wg_batch *);
template int conv_small_flush<float>(::ptl_wg_batch *);

template int conv_small<half_t>(const ConvTileDesc &, const void *, const void *, void *);
template int conv_small<float>(const ConvTileDesc &, const void *, const void *, void *);
template int conv_small_wg<half_t>(const ConvTileDesc &, const void *, const void *, void *, bool);
template int conv_small_wg<float>(const ConvTileDesc &, const void *, const void *, void *, bool);
template int conv_small_bw<half_t>(const ConvTileDesc &, const ConvTileDesc &, const void *, const void *, const void *,
                                   void *, void *, bool);
template int conv_small_bw<float>(const ConvTileDesc &, const ConvTileDesc &, const void *, const void *, const void *,
                                  void *, void *, bool);

}  // namespace ptl
