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
#include "ptl_host.hpp"

namespace ptl {
namespace {

constexpr int CS_NT = 1024, CS_WAVES = CS_NT / 64;
constexpr int CS_ITEMS = 32;                      // wave-wide load items per workgroup, at most
constexpr int CS_IN_MAX = CS_ITEMS / CS_WAVES;  // input pieces per thread

struct ConvSmallArgs {
    const half_t *X, *Wt;
    half_t *Y;
    int Cin, Cout, Hin, Win, Ho, Wo, s, padU, padL;
    int R, tiles_per_img;   // output rows per workgroup
    int RR, TW, POS;        // input rows of a tile, padded row width, RR * TW
    int items;              // wave-wide load items: (channel block, column group, block of 8 rows)
    int halo_chunks, halo_w;  // zero chunks of a tile: channel blocks x rows x halo columns; halo columns per row
    unsigned magic_halo_w, magic_rr;
    int f_chunks, f_inner;  // 16-byte pieces of the filter tensor [outer][inner][9]; inner dimension
    int f_transposed;       // 0: outer = filter, inner = channel; 1: outer = channel, inner = filter, taps flipped
    unsigned magic_inner9, magic_wo;
    int b_pitch, f_bytes;   // bytes per filter row in LDS, bytes of the filter tile
    int pgroups, mshift;    // jobs = groups of 32 pixels x (1 << mshift) blocks of 32 filters
    // per item: element offset into the sample (first channel, first tile row, column group), half offset into the
    // LDS tile, first tile row | first channel << 8
    int item_g[CS_ITEMS], item_l[CS_ITEMS], item_rc[CS_ITEMS];
};

union Piece {
    uint4 v;
    half_t e[8];
};

template <int CINP, int F_MAX>
__global__ __launch_bounds__(CS_NT) void conv_small_kernel(const ConvSmallArgs a) {
    extern __shared__ __attribute__((aligned(16))) char smem[];
    char *F = smem;
    half_t *T = reinterpret_cast<half_t *>(smem + a.f_bytes);  // [CINP / 8][POS][8]
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int b = blockIdx.x / a.tiles_per_img, y0 = (blockIdx.x - b * a.tiles_per_img) * a.R;
    const int iy0 = y0 * a.s - a.padU;

    // ---- all global loads first
    Piece xin[CS_IN_MAX];
    const int lrow = lane >> 3, lch = lane & 7;
    const half_t *xs = a.X + ((size_t)b * a.Cin + lch) * a.Hin * a.Win + (iy0 + lrow) * a.Win;
#pragma unroll
    for (int k = 0; k < CS_IN_MAX; ++k) {
        const int item = wave + CS_WAVES * k;
        xin[k].v = make_uint4(0, 0, 0, 0);
        if (item < a.items) {
            const int rc = a.item_rc[item], rr = (rc & 255) + lrow, ch = (rc >> 8) + lch, iy = iy0 + rr;
            if (rr < a.RR && ch < a.Cin && iy >= 0 && iy < a.Hin)
                xin[k].v = *reinterpret_cast<const uint4 *>(xs + a.item_g[item]);
        }
    }
    Piece fin[F_MAX];
#pragma unroll
    for (int k = 0; k < F_MAX; ++k) {
        const int q = tid + CS_NT * k;
        if (q < a.f_chunks) fin[k].v = reinterpret_cast<const uint4 *>(a.Wt)[q];
    }

    // channels the tensor does not have must read as zeros on the filter side too (0 x garbage is not 0)
    if (a.Cin < CINP) {
        for (int i = tid; i < a.f_bytes / 16; i += CS_NT) reinterpret_cast<uint4 *>(F)[i] = make_uint4(0, 0, 0, 0);
        __syncthreads();
    }
    // ---- halo columns of the tile: whole chunks of zeros
    for (int i = tid; i < a.halo_chunks; i += CS_NT) {
        const int row = fast_div(i, a.magic_halo_w), hc = i - row * a.halo_w;  // row = channel block * RR + tile row
        const int cb = fast_div(row, a.magic_rr), rr = row - cb * a.RR;
        const int col = hc < a.padL ? hc : a.Win + hc;
        reinterpret_cast<uint4 *>(T)[cb * a.POS + rr * a.TW + col] = make_uint4(0, 0, 0, 0);
    }
    // ---- input pieces -> [channel block][row][column] chunks
    half_t *tl = T + lrow * a.TW * 8 + lch;
#pragma unroll
    for (int k = 0; k < CS_IN_MAX; ++k) {
        const int item = wave + CS_WAVES * k;
        if (item < a.items && (a.item_rc[item] & 255) + lrow < a.RR) {
            half_t *row = tl + a.item_l[item];
#pragma unroll
            for (int j = 0; j < 8; ++j) row[j * 8] = xin[k].e[j];
        }
    }
    // ---- filter pieces -> [filter][tap][channel]: element (outer, inner, tap) of the dense tensor goes to
    // (filter, channel) = (outer, inner), or (inner, outer) with the taps flipped; the address moves with the indices
    {
        const int step_tap = a.f_transposed ? -CINP * 2 : CINP * 2;
        const int step_inner = (a.f_transposed ? a.b_pitch : 2) - 9 * step_tap;  // after the ninth tap step: tap 0, inner + 1
        const int step_outer = (a.f_transposed ? 2 : a.b_pitch) - a.f_inner * (a.f_transposed ? a.b_pitch : 2);
#pragma unroll
        for (int k = 0; k < F_MAX; ++k) {
            const int q = tid + CS_NT * k;
            if (q < a.f_chunks) {
                const int e0 = q * 8;
                const int outer = fast_div(e0, a.magic_inner9), rem = e0 - outer * a.f_inner * 9;
                int inner = (rem * 7282) >> 16;  // rem / 9 for rem < 2^15
                int tap = rem - inner * 9;
                const int m = a.f_transposed ? inner : outer, c = a.f_transposed ? outer : inner;
                int at = m * a.b_pitch + ((a.f_transposed ? 8 - tap : tap) * CINP + c) * 2;
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    *reinterpret_cast<half_t *>(F + at) = fin[k].e[j];
                    at += step_tap;
                    if (++tap == 9) {
                        tap = 0;
                        at += step_inner;
                        if (++inner == a.f_inner) {
                            inner = 0;
                            at += step_outer;
                        }
                    }
                }
            }
        }
    }
    __syncthreads();

    // ---- jobs: 32 pixels x 32 filters
    const int kg = lane >> 5, lr = lane & 31;
    const int npix = min(a.R, a.Ho - y0) * a.Wo, jobs = a.pgroups << a.mshift;
    const uint4 *T4 = reinterpret_cast<const uint4 *>(T);
    const size_t plane = (size_t)a.Ho * a.Wo;
    for (int job = wave; job < jobs; job += CS_NT / 64) {
        const int pg = job >> a.mshift, mb = job - (pg << a.mshift);
        if (pg * 32 >= npix) break;
        const int p = min(pg * 32 + lr, npix - 1);
        const int py = fast_div(p, a.magic_wo), px = p - py * a.Wo;
        const uint4 *prow = T4 + (py * a.TW + px) * a.s + kg * a.POS;
        const char *frow = F + (mb * 32 + lr) * a.b_pitch + kg * 16;
        f32x16 acc;
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[v] = 0.f;
#pragma unroll
        for (int ks = 0; ks < CINP / 16; ++ks) {
            const uint4 *pk = prow + 2 * ks * a.POS;
#pragma unroll
            for (int ky = 0; ky < 3; ++ky) {
                const uint4 *pr = pk + ky * a.TW;
#pragma unroll
                for (int kx = 0; kx < 3; ++kx) {
                    const uint4 pf = pr[kx];
                    const uint4 ff = *reinterpret_cast<const uint4 *>(frow + ((ky * 3 + kx) * CINP + ks * 16) * 2);
                    mfma_step<half_t>(acc, ff, pf);
                }
            }
        }
        if (pg * 32 + lr < npix) {
            half_t *out = a.Y + (((size_t)b * a.Cout + mb * 32 + 4 * kg) * a.Ho + y0 + py) * a.Wo + px;
            const int left = a.Cout - mb * 32 - 4 * kg;  // filters from this lane's first one
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int f = 8 * (v >> 2) + (v & 3);
                if (f < left) out[f * plane] = (half_t)acc[v];
            }
        }
    }
}

template <int CINP, int F_MAX>
int launch_small(const ConvSmallArgs &a, int tiles, size_t lds, hipStream_t s) {
    state().last_conv_resident = 2;
    auto kern = conv_small_kernel<CINP, F_MAX>;
    static bool attr_set = false;
    if (!attr_set) {
        if (!hip_ok(hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, 150 * 1024),
                    "hipFuncSetAttribute"))
            return 2;
        attr_set = true;
    }
    hipLaunchKernelGGL(kern, dim3(tiles), dim3(CS_NT), lds, s, a);
    return hip_ok(hipGetLastError(), "small convolution launch") ? 0 : 2;
}

}  // namespace

int conv_small(const ConvTileDesc &d, const void *X, const void *Wt, void *Y) {
    State &st = state();
    if (st.gemm_path != 0 && st.gemm_path != 6) return -1;  // (the other values select one of the other routes)
    if (d.in_hwc || d.KH != 3 || d.KW != 3 || d.sh != d.sw || d.sh < 1 || d.sh > 2) return -1;
    if (d.Cin > 64 || d.Cout > 64 || d.Win % 8 != 0 || d.x_sy != d.Win) return -1;
    if (d.x_sc != (long long)d.Hin * d.Win || d.x_sb != (long long)d.Cin * d.Hin * d.Win) return -1;
    if (d.padU < 0 || d.padU > 2 || d.padL < 0 || d.padL > 2 || d.padD < 0 || d.padR < 0 || d.padR > 8) return -1;
    if (reinterpret_cast<uintptr_t>(X) % 16 || reinterpret_cast<uintptr_t>(Wt) % 16) return -1;
    const long long f_elems = (long long)d.Cout * d.Cin * 9;
    if (f_elems % 8 != 0) return -1;
    ConvSmallArgs a = {};
    // dense filter tensor [outer][inner][3][3]: forward (filter, channel), or the input gradient's view of it
    if (d.w_base == 0 && d.w_sm == d.Cin * 9 && d.w_sc == 9 && d.w_sy == 3 && d.w_sx == 1) {
        a.f_transposed = 0;
        a.f_inner = d.Cin;
    } else if (d.w_base == 8 && d.w_sm == 9 && d.w_sc == d.Cout * 9 && d.w_sy == -3 && d.w_sx == -1) {
        a.f_transposed = 1;
        a.f_inner = d.Cout;
    } else {
        return -1;
    }
    const int s = d.sh, TW = d.Win + d.padL + d.padR, THP = d.Hin + d.padU + d.padD;
    if ((d.Wo - 1) * s + 3 > TW || (d.Ho - 1) * s + 3 > THP || d.Wo >= 65536 || d.Ho * d.Wo >= 65536) return -1;
    const int cinp = d.Cin <= 16 ? 16 : d.Cin <= 32 ? 32 : 64, cblocks = cinp / 8;
    const int mblocks = (d.Cout + 31) / 32;
    // rows per workgroup: the whole image, halved while that leaves the four waves a job each and the chip is not full
    int R = d.Ho;
    auto jobs_of = [&](int r) { return ((r * d.Wo + 31) / 32) * mblocks; };
    while ((long long)d.batch * ((d.Ho + R - 1) / R) < st.num_cu && R % 2 == 0 && jobs_of(R / 2) >= 4) R /= 2;
    auto items_of = [&](int r) { return cblocks * (d.Win / 8) * ((((r - 1) * s + 3) + 7) / 8); };
    auto lds_of = [&](int r) { return (size_t)cblocks * ((r - 1) * s + 3) * TW * 16; };
    const int pitch = 9 * cinp * 2 + 16;
    const size_t f_bytes = (size_t)mblocks * 32 * pitch;
    while (R > 1 && (items_of(R) > CS_ITEMS || f_bytes + lds_of(R) > 150 * 1024)) R = (R + 1) / 2;
    if (items_of(R) > CS_ITEMS || f_bytes + lds_of(R) > 150 * 1024) return -1;
    const long long tiles = (long long)d.batch * ((d.Ho + R - 1) / R);
    // beyond a few workgroups per CU the persistent kernels (filters loaded once per workgroup) are ahead
    if (st.gemm_path != 6 && tiles > 4LL * st.num_cu) return -1;
    if (tiles >= (1LL << 31) / 256) return -1;
    a.X = reinterpret_cast<const half_t *>(X);
    a.Wt = reinterpret_cast<const half_t *>(Wt);
    a.Y = reinterpret_cast<half_t *>(Y);
    a.Cin = d.Cin; a.Cout = d.Cout; a.Hin = d.Hin; a.Win = d.Win; a.Ho = d.Ho; a.Wo = d.Wo;
    a.s = s; a.padU = d.padU; a.padL = d.padL;
    a.R = R; a.tiles_per_img = (d.Ho + R - 1) / R;
    a.RR = (R - 1) * s + 3; a.TW = TW; a.POS = a.RR * TW;
    const int G = d.Win / 8, RR8 = (a.RR + 7) / 8;
    a.items = cblocks * G * RR8;
    for (int item = 0; item < a.items; ++item) {
        const int rblk = item % RR8, t = item / RR8, g = t % G, cb = t / G;
        a.item_g[item] = (cb * 8 * d.Hin + rblk * 8) * d.Win + 8 * g;
        a.item_l[item] = ((cb * a.POS + rblk * 8 * TW) + d.padL + 8 * g) * 8;
        a.item_rc[item] = (rblk * 8) | ((cb * 8) << 8);
    }
    a.halo_w = TW - d.Win;
    a.halo_chunks = cblocks * a.RR * a.halo_w;
    a.magic_halo_w = magic_of(a.halo_w);
    a.magic_rr = magic_of(a.RR);
    a.f_chunks = (int)(f_elems / 8);
    a.magic_inner9 = magic_of(a.f_inner * 9);
    a.magic_wo = magic_of(d.Wo);
    a.b_pitch = pitch; a.f_bytes = (int)f_bytes;
    a.pgroups = (R * d.Wo + 31) / 32; a.mshift = mblocks - 1;
    if (f_elems >= 65536 || a.f_inner * 9 >= 65536) return -1;  // (quotients by reciprocal multiplication)
    const size_t lds = f_bytes + lds_of(R);
    const int per_thread = (a.f_chunks + CS_NT - 1) / CS_NT;
    if (a.halo_chunks >= 65536 || a.RR * cblocks >= 65536) return -1;
    if (cinp == 16) {
        if (per_thread <= 1) return launch_small<16, 1>(a, (int)tiles, lds, st.stream);
        if (per_thread <= 2) return launch_small<16, 2>(a, (int)tiles, lds, st.stream);
        return -1;
    }
    if (cinp == 32) {
        if (per_thread <= 2) return launch_small<32, 2>(a, (int)tiles, lds, st.stream);
        if (per_thread <= 3) return launch_small<32, 3>(a, (int)tiles, lds, st.stream);
        return -1;
    }
    if (per_thread <= 3) return launch_small<64, 3>(a, (int)tiles, lds, st.stream);
    if (per_thread <= 5) return launch_small<64, 5>(a, (int)tiles, lds, st.stream);
    return -1;
}

}  // namespace ptl
