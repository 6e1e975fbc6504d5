// Convolution as a sum over filter taps on the look-up-free pipelined GEMM (unit stride, channel counts that
// are multiples of a 128-byte slab: 64 halves / 32 floats; channel-major or channel-minor tensors).
//
//   Y[(b,y,x)][co] = sum over taps (ky,kx) and channels c of  Xp[b][c][y+ky][x+kx] * W[co][c][ky][kx]
//
// Two small passes prepare the operands in the library's scratch memory:
//   * the input, zero-padded and channel-blocked as [c/VEC][b][y][x][VEC] (16-byte chunks = VEC consecutive
//     channels of one position).  For a fixed tap this IS a plain [pixel][channel] matrix: pixel (b,y,x) starts
//     at a fixed offset, chunk j of a slab sits j channel-block planes further, and moving to another tap adds
//     one constant to every address - no border tests, no im2col;
//   * the filters as [co][tap][c], so that k = (tap, c) is contiguous.
// The GEMM kernel then runs its ordinary slab loop over k = taps x channels with one pointer jump per tap.
// A channel-minor input [b][y][x][c] only needs its zero halo: [b][yp][xp][c] is the same kind of matrix with
// the channels of a pixel contiguous (a slab of k is 128 consecutive bytes) and a tap shift of C elements.
// The input gradient is the same product over the (padded) output gradient with flipped, transposed filters;
// the filter pass reads them through the strides of the descriptor.
#include "ptl_conv_tile.hpp"
#include "ptl_gemm_async.hpp"
#include "ptl_structs.h"

namespace ptl {

static ::ptl_conv_cache *g_cache_fill = nullptr;
static const ::ptl_conv_cache *g_cache_use = nullptr;
static const ::ptl_conv_cache *g_cache_in = nullptr;
static ::ptl_conv_cache *g_cache_out = nullptr;
void conv_cache_set(::ptl_conv_cache *fill, const ::ptl_conv_cache *use) {
    g_cache_fill = fill;
    g_cache_use = use;
}
void conv_cache_chain(const ::ptl_conv_cache *in, ::ptl_conv_cache *out) {
    g_cache_in = in;
    g_cache_out = out;
}

// The cached copy, if the call in progress was given one that fits this layer: `chunks` 16-byte pieces (margin
// included) of the blocked, padded input of `d`.
static const uint4 *cached_input(const ConvTileDesc &d, int Hp, int Wp, long long chunks,
                                 const ::ptl_conv_cache *c = g_cache_use) {
    if (!c || !c->valid || !c->buf || c->bytes < (size_t)chunks * 16) return nullptr;
    const int want[6] = {d.batch, d.Cin, Hp, Wp, d.padU, d.padL};
    for (int i = 0; i < 6; ++i)
        if (c->geometry[i] != want[i]) return nullptr;
    return reinterpret_cast<const uint4 *>(c->buf);
}

// in: [b][C][H][W] (strides sb, sc; rows contiguous) -> out: [C/VEC][B][Hp][Wp] chunks, zero halo.
template <typename T>
__device__ inline void chw_to_blocked_padded(unsigned block, const T *__restrict__ in, uint4 *__restrict__ out, int B,
                                             int H, int W, int Hp, int Wp, int padU, int padL, long long sb,
                                             long long sc, int cblocks, long long total) {
    constexpr int VEC = 16 / (int)sizeof(T);
    // (the host keeps the copy below 2^31 bytes: 32-bit index arithmetic)
    const unsigned i = block * 256u + threadIdx.x;
    if (i >= total) return;
    unsigned r = i / (unsigned)Wp;
    const int xp = (int)(i - r * Wp);
    const unsigned r2 = r / (unsigned)Hp;
    const int yp = (int)(r - r2 * Hp);
    const int cb = (int)(r2 / (unsigned)B), b = (int)(r2 - (unsigned)cb * B);
    const int y = yp - padU, x = xp - padL;
    union {
        uint4 v;
        T e[VEC];
    } u;
    if (cb < cblocks && y >= 0 && y < H && x >= 0 && x < W) {  // beyond the last block: zero margin
        const T *src = in + b * sb + (long long)(cb * VEC) * sc + (long long)y * W + x;
#pragma unroll
        for (int e = 0; e < VEC; ++e) u.e[e] = src[e * sc];
    } else {
        u.v = make_uint4(0, 0, 0, 0);
    }
    out[i] = u.v;
}

template <typename T>
__global__ __launch_bounds__(256) void chw_to_blocked_padded_kernel(const T *__restrict__ in, uint4 *__restrict__ out,
                                                                    int B, int H, int W, int Hp, int Wp, int padU,
                                                                    int padL, long long sb, long long sc,
                                                                    int cblocks, long long total) {
    chw_to_blocked_padded<T>(blockIdx.x, in, out, B, H, W, Hp, Wp, padU, padL, sb, sc, cblocks, total);
}

// Launches the padded, blocked copy of X ([b][C][H][W]) with `margin` zero chunks after it.
template <typename T>
static int blocked_padded_copy(const T *X, uint4 *xb, const ConvTileDesc &d, int Hp, int Wp, long long margin) {
    State &st = state();
    constexpr int VEC = 16 / (int)sizeof(T);
    const int cblocks = d.Cin / VEC;
    const long long planes = (long long)cblocks * d.batch, chunks = planes * Hp * Wp;
    hipLaunchKernelGGL((chw_to_blocked_padded_kernel<T>), dim3((unsigned)((chunks + margin + 255) / 256)), dim3(256),
                       0, st.stream, X, xb, d.batch, d.Hin, d.Win, Hp, Wp, d.padU, d.padL, d.x_sb, d.x_sc, cblocks,
                       chunks + margin);
    return hip_ok(hipGetLastError(), "blocked layout launch") ? 0 : 2;
}

// in: [b][H][W][C] as 16-byte chunks (cblocks per pixel) -> out: [b][Hp][Wp][C], zero halo.
__device__ inline void hwc_to_padded(unsigned block, const uint4 *__restrict__ in, uint4 *__restrict__ out, int B,
                                     int H, int W, int Hp, int Wp, int padU, int padL, int cblocks, long long total) {
    const unsigned i = block * 256u + threadIdx.x;
    if (i >= total) return;
    const unsigned pix = i / (unsigned)cblocks, cc = i - pix * cblocks;
    const unsigned r = pix / (unsigned)Wp, b = r / (unsigned)Hp;
    const int y = (int)(r - b * Hp) - padU, x = (int)(pix - r * Wp) - padL;
    uint4 v = make_uint4(0, 0, 0, 0);
    if (b < (unsigned)B && y >= 0 && y < H && x >= 0 && x < W) v = in[((b * H + y) * W + x) * cblocks + cc];
    out[i] = v;  // (beyond the last sample: zero margin)
}

__global__ __launch_bounds__(256) void hwc_to_padded_kernel(const uint4 *__restrict__ in, uint4 *__restrict__ out, int B,
                                                            int H, int W, int Hp, int Wp, int padU, int padL,
                                                            int cblocks, long long total) {
    hwc_to_padded(blockIdx.x, in, out, B, H, W, Hp, Wp, padU, padL, cblocks, total);
}

// out[m][tap][c] = W[base + m*sm + c*sc + ky*sy + kx*sx]
template <typename T>
__device__ inline void filters_tap_major(unsigned block, const T *__restrict__ w, T *__restrict__ out, int C, int KW,
                                         int taps, long long base, long long sm, long long sc, long long sy,
                                         long long sx, long long total) {
    const long long i = (long long)block * 256 + threadIdx.x;
    if (i >= total) return;
    const int c = (int)(i % C);
    const long long r = i / C;
    const int t = (int)(r % taps);
    const long long m = r / taps;
    out[i] = w[base + m * sm + c * sc + (t / KW) * sy + (t % KW) * sx];
}

// Both layout passes of the forward / input-gradient route in one launch: the first `copy_blocks` workgroups
// write the padded, blocked input, the rest the tap-major filters.
struct TapPrepArgs {
    const void *in;
    uint4 *xb;
    int B, H, W, Hp, Wp, padU, padL, cblocks, hwc;
    long long sb, sc, xb_total;
    unsigned copy_blocks;
    const void *w;
    void *wr;
    int C, KW, taps;
    long long w_base, w_sm, w_sc, w_sy, w_sx, wr_total;
    // the backward pass's two other passes, in front of the first: the blocked copy of the output gradient
    // (embed_blocks workgroups, see halo_embed_chunk) and zero_n chunks of zeros at zero_at (zero_blocks workgroups)
    const void *e_in;
    uint4 *e_out;
    int e_Ho, e_Wo, e_Hp, e_Wp, e_pu, e_pl;
    long long e_sb, e_sc;
    unsigned e_P, e_pstride, e_total, embed_blocks;
    uint4 *zero_at;
    unsigned zero_n, zero_blocks;
};
template <typename T>
__global__ __launch_bounds__(256) void tap_prepare_kernel(const TapPrepArgs a) {
    unsigned bid = blockIdx.x;
    if (bid < a.embed_blocks) {
        const unsigned i = bid * 256u + threadIdx.x;
        if (i < a.e_total)
            halo_embed_chunk(i, reinterpret_cast<const half_t *>(a.e_in), a.e_out, a.e_Ho, a.e_Wo, a.e_Hp, a.e_Wp, a.e_pu,
                             a.e_pl, a.e_sb, a.e_sc, a.e_P, a.e_pstride);
        return;
    }
    bid -= a.embed_blocks;
    if (bid < a.zero_blocks) {
        const unsigned i = bid * 256u + threadIdx.x;
        if (i < a.zero_n) a.zero_at[i] = make_uint4(0, 0, 0, 0);
        return;
    }
    bid -= a.zero_blocks;
    if (bid < a.copy_blocks && a.hwc)
        hwc_to_padded(bid, reinterpret_cast<const uint4 *>(a.in), a.xb, a.B, a.H, a.W, a.Hp, a.Wp, a.padU, a.padL,
                      a.cblocks, a.xb_total);
    else if (bid < a.copy_blocks)
        chw_to_blocked_padded<T>(bid, reinterpret_cast<const T *>(a.in), a.xb, a.B, a.H, a.W, a.Hp, a.Wp, a.padU,
                                 a.padL, a.sb, a.sc, a.cblocks, a.xb_total);
    else
        filters_tap_major<T>(bid - a.copy_blocks, reinterpret_cast<const T *>(a.w), reinterpret_cast<T *>(a.wr),
                             a.C, a.KW, a.taps, a.w_base, a.w_sm, a.w_sc, a.w_sy, a.w_sx, a.wr_total);
}

__global__ __launch_bounds__(256) void zero_chunks_kernel(uint4 *__restrict__ p, unsigned n) {
    const unsigned i = blockIdx.x * 256u + threadIdx.x;
    if (i < n) p[i] = make_uint4(0, 0, 0, 0);
}

template <typename T>
int conv_taps(const ConvTileDesc &d, const void *X, const void *Wt, void *Y, const OutMap &c) {
    State &st = state();
    constexpr int ES = (int)sizeof(T), VEC = 16 / ES, SK = 128 / ES;
    const bool hwc = d.in_hwc != 0;
    if (d.sh != 1 || d.sw != 1 || d.Cin % SK) return -1;
    if (hwc ? reinterpret_cast<uintptr_t>(X) % 16 != 0 : d.x_sy != d.Win) return -1;
    const int taps = d.KH * d.KW;
    int Hp, Wp;
    conv_padded_grid(d, &Hp, &Wp);
    if (!conv_output_fits_pads(d) || taps < 2) return -1;
    const int cblocks = d.Cin / VEC;
    const long long plane = (long long)Hp * Wp * VEC;            // elements of one (channel block, sample) plane
    const long long xb_elems = (long long)cblocks * d.batch * plane;
    const long long wr_elems = (long long)d.Cout * taps * d.Cin;
    const long long npix = (long long)d.batch * d.Ho * d.Wo;
    if (xb_elems * ES >= ((long long)1 << 31) || npix >= ((long long)1 << 31) || wr_elems >= ((long long)1 << 31))
        return -1;
    if (st.gemm_path == 2) return -1;
    // (only with at least 64 filters: narrower products fall to the GEMM's slim tiles, where the direct kernel wins)
    // and from about a thousand output pixels: measured at 128..512 channels, batch 8..32, the two layout passes pay
    // from 1568 pixels on (12.6 against 24.2 us for 128 -> 128 on 14x14 at batch 8, 35.8 against 74.5 us for
    // 512 -> 512 on 7x7 at batch 32) and do not at 392 (20.5 against 14.8 us for 256 -> 256 on 7x7 at batch 8).
    const bool forced = st.gemm_path == 3 || st.gemm_path == 5;
    // (32 filters - the input gradient of a layer with 32 channels - only on the resident-tile kernel below)
    const bool slim = d.Cout < 64 && !(ES == 2 && !hwc && d.Cout % 32 == 0 && conv_halo_fits(d, Hp, Wp));
    if (!forced && (slim || npix < 1024)) return -1;
    // 3x3 fp16 layers keep the input tile in LDS for all nine taps (ptl_conv_halo.hip): the tap-sum GEMM fetches it
    // once per tap.  Measured at batch 128..512, forward: 64 -> 64 on 56x56 63 against 96 us, 128 -> 128 on 28x28
    // 52 against 76, 256 -> 256 on 28x28 295 against 372, 512 -> 512 on 14x14 273 against 293.  Its workgroups are
    // persistent over whole tiles (256 positions x 64 / 128 filters x all channels), so it needs enough tiles: below
    // about 48 (32 for a single 64-channel slab) the GEMM, which splits the contraction, is faster (14.0 against
    // 19.0 us for 128 -> 128 on 28x28 at batch 8, 35.8 against 56.5 us for 512 -> 512 on 7x7 at batch 32).
    const long long halo_tiles = ((long long)d.batch * Hp * Wp + 255) / 256 * ((d.Cout + 127) / 128);
    const bool halo_pays = halo_tiles >= 48 || (d.Cin == 64 && halo_tiles >= 32);
    // channel-minor tensors: the same kernel reads them in place (no padded copy; the filters too when they are
    // tap-major as they lie, which the forward pass's are)
    if (ES == 2 && hwc && conv_halo_hwc_fits(d, X, Y) && (st.gemm_path == 5 || (st.gemm_path == 0 && halo_pays))) {
        const void *wr = Wt;
        if (!(d.w_base == 0 && d.w_sc == 1 && d.w_sx == d.Cin && d.w_sy == d.KW * d.Cin && d.w_sm == taps * d.Cin &&
              reinterpret_cast<uintptr_t>(Wt) % 16 == 0)) {
            char *buf = static_cast<char *>(scratch((size_t)wr_elems * ES + 256));
            if (!buf) return 2;
            TapPrepArgs p = {};
            p.copy_blocks = 0;
            p.w = Wt;
            p.wr = buf;
            p.C = d.Cin; p.KW = d.KW; p.taps = taps;
            p.w_base = d.w_base; p.w_sm = d.w_sm; p.w_sc = d.w_sc; p.w_sy = d.w_sy; p.w_sx = d.w_sx;
            p.wr_total = wr_elems;
            hipLaunchKernelGGL((tap_prepare_kernel<T>), dim3((unsigned)((wr_elems + 255) / 256)), dim3(256), 0, st.stream, p);
            if (!hip_ok(hipGetLastError(), "layout launch")) return 2;
            wr = buf;
        }
        st.last_conv_resident = 1;
        return conv_halo_hwc_launch(d, X, wr, Y);
    }
    const bool halo = ES == 2 && !hwc && conv_halo_fits(d, Hp, Wp) && (long long)d.batch * Hp * Wp < ((long long)1 << 31) &&
                      (st.gemm_path == 5 || (st.gemm_path == 0 && halo_pays));
    if (!halo && d.Cout < 64 && st.gemm_path != 3) return -1;  // (the tap-sum GEMM has no tile for fewer than 64 filters)
    // chunks read past the end: the resident-tile kernel's reach, or the window of the last sample's last pixels
    const long long margin = halo ? conv_halo_margin() : ((long long)(d.KH - 1) * Wp + d.KW) * (hwc ? cblocks : 1);
    // the blocked input goes to the caller's buffer when the call brought one (the weight gradient of the layer
    // reads the same copy), else to scratch memory like the filters
    const size_t xb_bytes = (size_t)(xb_elems + margin * VEC) * ES;
    // a copy the call was handed (left by the layer that produced the input): nothing to copy
    const uint4 *given = halo && g_cache_in ? cached_input(d, Hp, Wp, xb_elems / VEC + margin, g_cache_in) : nullptr;
    ::ptl_conv_cache *fill = given ? nullptr : g_cache_fill;
    const bool keep = halo && fill && fill->buf && fill->bytes >= xb_bytes && reinterpret_cast<uintptr_t>(fill->buf) % 16 == 0;
    char *buf = static_cast<char *>(scratch(((keep || given) ? 0 : xb_bytes) + (size_t)wr_elems * ES + 512));
    if (!buf) return 2;
    uint4 *xb = given ? const_cast<uint4 *>(given) : reinterpret_cast<uint4 *>(keep ? static_cast<char *>(fill->buf) : buf);
    T *wr = reinterpret_cast<T *>((keep || given) ? buf : buf + ((xb_bytes + 255) & ~(size_t)255));
    if (keep) {
        const int geo[6] = {d.batch, d.Cin, Hp, Wp, d.padU, d.padL};
        for (int i = 0; i < 6; ++i) fill->geometry[i] = geo[i];
        fill->valid = 1;
    }
    {
        TapPrepArgs p = {};
        p.in = X;
        p.xb = xb;
        p.B = d.batch; p.H = d.Hin; p.W = d.Win; p.Hp = Hp; p.Wp = Wp; p.padU = d.padU; p.padL = d.padL;
        p.cblocks = cblocks;
        p.hwc = hwc;
        p.sb = d.x_sb; p.sc = d.x_sc;
        p.xb_total = xb_elems / VEC + margin;
        p.copy_blocks = given ? 0u : (unsigned)((p.xb_total + 255) / 256);
        p.w = Wt;
        p.wr = wr;
        p.C = d.Cin; p.KW = d.KW; p.taps = taps;
        p.w_base = d.w_base; p.w_sm = d.w_sm; p.w_sc = d.w_sc; p.w_sy = d.w_sy; p.w_sx = d.w_sx;
        p.wr_total = wr_elems;
        hipLaunchKernelGGL((tap_prepare_kernel<T>), dim3(p.copy_blocks + (unsigned)((wr_elems + 255) / 256)), dim3(256),
                           0, st.stream, p);
        if (!hip_ok(hipGetLastError(), "layout launch")) return 2;
    }

    st.last_conv_resident = halo;
    if (halo) {
        // the output once more as the next layer's blocked, padded input, when the call brought a prepared buffer
        // for it (geometry: batch, channels, padded height and width, top and left padding of that layer)
        ::ptl_conv_cache *out = g_cache_out;
        HaloOutCopy oc = {};
        if (out && out->buf && reinterpret_cast<uintptr_t>(out->buf) % 16 == 0 && out->geometry[0] == d.batch &&
            out->geometry[1] == d.Cout && d.Cout % 8 == 0 && out->geometry[2] > 0 && out->geometry[3] > 0 &&
            out->bytes >= ((size_t)(d.Cout / 8) * d.batch * out->geometry[2] * out->geometry[3] + (size_t)conv_halo_margin()) * 16) {
            oc.buf = out->buf;
            oc.Hp = out->geometry[2]; oc.Wp = out->geometry[3]; oc.padU = out->geometry[4]; oc.padL = out->geometry[5];
            oc.relu = out->relu != 0;
        }
        int rc = conv_halo_launch(d, xb, wr, Y, Hp, Wp, 0, oc.buf ? &oc : nullptr);
        if (rc == -1 && oc.buf) {  // (the copy does not fit this layer's output: the layer without it)
            oc.buf = nullptr;
            rc = conv_halo_launch(d, xb, wr, Y, Hp, Wp);
        }
        if (rc == 0 && oc.buf) out->valid = 1;
        return rc;
    }

    GemmArgs q = {};
    q.A = xb;
    q.B = wr;
    q.C = Y;
    q.N = (int)npix;
    q.M = d.Cout;
    q.K = taps * d.Cin;
    q.a.HL = q.a.WL = q.b.HL = q.b.WL = 1;
    // row = pixel (b, y, x) of the padded input
    q.a.row = {};
    q.a.row.n = q.N;
    q.a.row.d1 = d.Ho;
    q.a.row.d0 = d.Wo;
    // per sample / padded row / pixel; a 16-byte chunk further along k is one block plane on (channel-major) or
    // the next 16 bytes (channel-minor)
    const long long sample = (long long)Hp * Wp * d.Cin, pix_shift = hwc ? d.Cin : VEC;
    const long long kstride = hwc ? 1 : (long long)d.batch * plane / VEC;  // per channel
    if (kstride >= ((long long)1 << 31) || sample >= ((long long)1 << 31)) return -1;
    q.a.row.o2 = hwc ? (int)sample : (int)plane;
    q.a.row.o1 = Wp * (int)pix_shift;
    q.a.row.o0 = (int)pix_shift;
    q.a.k = axis_plain(q.K, (int)kstride);
    q.a.mode = FILL_VEC_K;
    q.b.row = axis_plain(d.Cout, q.K);
    q.b.k = axis_plain(q.K, 1);
    q.b.mode = FILL_VEC_K;
    q.c = c;
    q.taps = taps;
    q.slabs_per_tap = d.Cin / SK;
    q.tap_kw = d.KW;
    const long long tap_span = (long long)q.slabs_per_tap * SK * kstride * ES;  // what the slabs of a tap advance A by
    q.tap_jump_x = pix_shift * ES - tap_span;
    q.tap_jump_y = (long long)(Wp - (d.KW - 1)) * pix_shift * ES - tap_span;
    return gemm_async<T>(q);
}


// ---------------------------------------------------------------------------------------------------------
// Weight gradient the same way: for every tap (ky,kx)
//   dW[co][c][ky][kx] = sum over padded positions pp of all samples of  dYp[co][pp] * Xp[c][pp + ky*Wp + kx]
// with dYp the output gradient embedded in the padded grid (zero where no output pixel sits) and Xp the
// blocked, padded input: per tap a [co][pp] x [pp][c] product whose second operand is the SAME matrix
// shifted by a constant.  One launch covers all taps and k splits (grid.y), one kernel adds the partial sums.

// out[co][k], k = (b, yp, xp) flattened and padded to Kr: dY[b][co][yp][xp] inside the output, else zero.
// One thread per 16 bytes of the destination.
template <typename T>
__global__ __launch_bounds__(256) void embed_gradient_kernel(const T *__restrict__ dy, uint4 *__restrict__ out, int B,
                                                             int Cout, int Ho, int Wo, int Hp, int Wp, long long Kr,
                                                             long long total) {
    constexpr int VEC = 16 / (int)sizeof(T);
    // (the host keeps the copy below 2^31 bytes: 32-bit index arithmetic)
    const unsigned i = blockIdx.x * 256u + threadIdx.x;
    if (i >= total) return;
    const unsigned kv = (unsigned)(Kr / VEC);
    const int co = (int)(i / kv);
    const unsigned k0 = (i - (unsigned)co * kv) * VEC;
    unsigned r = k0 / (unsigned)Wp;
    int xp = (int)(k0 - r * Wp);
    long long b = r / (unsigned)Hp;
    int yp = (int)(r - (unsigned)b * Hp);
    union {
        uint4 v;
        T e[VEC];
    } u;
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
        u.e[e] = (b < B && yp < Ho && xp < Wo) ? dy[((b * Cout + co) * Ho + yp) * (long long)Wo + xp] : (T)0;
        if (++xp == Wp) {
            xp = 0;
            if (++yp == Hp) {
                yp = 0;
                ++b;
            }
        }
    }
    out[i] = u.v;
}

// Channel-minor twin: out[k][co] in 16-byte chunks (cv per position), k = (b, yp, xp) over the padded grid and
// up to krows; dY[b][yp][xp][co] inside the output, else zero.
__global__ __launch_bounds__(256) void embed_gradient_hwc_kernel(const uint4 *__restrict__ dy, uint4 *__restrict__ out,
                                                                 int B, int cv, int Ho, int Wo, int Hp, int Wp,
                                                                 long long total) {
    const unsigned i = blockIdx.x * 256u + threadIdx.x;
    if (i >= total) return;
    const unsigned k = i / (unsigned)cv, cc = i - k * cv;
    const unsigned r = k / (unsigned)Wp, b = r / (unsigned)Hp;
    const unsigned yp = r - b * Hp, xp = k - r * Wp;
    uint4 v = make_uint4(0, 0, 0, 0);
    if (b < (unsigned)B && yp < (unsigned)Ho && xp < (unsigned)Wo) v = dy[((b * Ho + yp) * Wo + xp) * cv + cc];
    out[i] = v;
}

// dW[(n*M + m)*taps + tap] = sum over the splits of ws[tap][split][n][m]; 64 outputs x 4 split groups per
// workgroup, four loads in flight per thread.
template <typename T>
__global__ __launch_bounds__(256) void taps_wg_reduce_kernel(const float *__restrict__ ws, T *__restrict__ dW,
                                                             long long total, int splits, int taps, int M,
                                                             int tap_major) {
    __shared__ float part[4][64];
    const int o = threadIdx.x & 63, sg = threadIdx.x >> 6, tap = blockIdx.y;
    const long long idx = (long long)blockIdx.x * 64 + o;
    float s = 0.f;
    if (idx < total) {
        const float *src = ws + (long long)tap * splits * total + idx;
        int z = sg;
        for (; z + 12 < splits; z += 16) {
            float v[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) v[u] = src[(long long)(z + u * 4) * total];
#pragma unroll
            for (int u = 0; u < 4; ++u) s += v[u];
        }
        for (; z < splits; z += 4) s += src[(long long)z * total];
    }
    part[sg][o] = s;
    __syncthreads();
    if (sg != 0 || idx >= total) return;
    s += part[1][o] + part[2][o] + part[3][o];
    // [n][m][tap] (channel-major filters) or [n][tap][m] (channel-minor)
    dW[tap_major ? ((idx / M) * taps + tap) * M + idx % M : idx * taps + tap] = (T)s;
}

template <typename T>
int conv_taps_wg(const ConvTileDesc &d, const void *X, const void *dY, void *dW) {
    State &st = state();
    constexpr int ES = (int)sizeof(T), VEC = 16 / ES, SK = 128 / ES;
    const bool hwc = d.in_hwc != 0;
    if (d.sh != 1 || d.sw != 1 || d.Cin % VEC) return -1;
    if constexpr (ES == 2) {
        // 3x3 channel-major layers: both operands channel-blocked, tiles resident in LDS for all taps
        int Hp, Wp;
        conv_padded_grid(d, &Hp, &Wp);
        if (!hwc && d.x_sy == d.Win && conv_halo_wg_fits(d, Hp, Wp) &&
            (st.gemm_path == 5 || (st.gemm_path == 0 && conv_halo_wg_preferred(d)))) {
            const long long P = (long long)d.batch * Hp * Wp, margin = conv_halo_wg_margin();
            const long long xb_chunks = (long long)(d.Cin / VEC) * P + margin;
            const long long gb_chunks = (long long)(d.Cout / VEC) * conv_halo_wg_gradient_stride(d, Hp, Wp);
            int S0 = 1, S1 = 1;
            const size_t ws_bytes = conv_halo_wg_partial_bytes(d, Hp, Wp, &S0, &S1);
            if (xb_chunks * 16 < ((long long)1 << 31) && gb_chunks * 16 < ((long long)1 << 31) &&
                ws_bytes <= ((size_t)1 << 30)) {
                char *buf = static_cast<char *>(scratch((size_t)(xb_chunks + gb_chunks) * 16 + 256));
                if (!buf) return 2;
                float *ws = workspace(ws_bytes);
                if (!ws) return 2;
                uint4 *xb = reinterpret_cast<uint4 *>(buf);
                char *gb = buf + (((size_t)xb_chunks * 16 + 255) & ~(size_t)255);
                // both layout passes in one launch (the blocked copy of the output gradient, and that of the input
                // unless the call was handed one)
                const long long gstride = conv_halo_wg_gradient_stride(d, Hp, Wp);
                const uint4 *kept = cached_input(d, Hp, Wp, xb_chunks);
                if (gstride < P) return -1;
                {
                    TapPrepArgs p = {};
                    p.e_in = dY;
                    p.e_out = reinterpret_cast<uint4 *>(gb);
                    p.e_Ho = d.Ho; p.e_Wo = d.Wo; p.e_Hp = Hp; p.e_Wp = Wp;
                    p.e_sb = (long long)d.Cout * d.Ho * d.Wo;
                    p.e_sc = (long long)d.Ho * d.Wo;
                    p.e_P = (unsigned)P;
                    p.e_pstride = (unsigned)gstride;
                    p.e_total = (unsigned)gb_chunks;
                    p.embed_blocks = (unsigned)((gb_chunks + 255) / 256);
                    if (!kept) {
                        p.in = X;
                        p.xb = xb;
                        p.B = d.batch; p.H = d.Hin; p.W = d.Win; p.Hp = Hp; p.Wp = Wp; p.padU = d.padU; p.padL = d.padL;
                        p.cblocks = d.Cin / VEC;
                        p.sb = d.x_sb; p.sc = d.x_sc;
                        p.xb_total = xb_chunks;
                        p.copy_blocks = (unsigned)((xb_chunks + 255) / 256);
                    }
                    hipLaunchKernelGGL((tap_prepare_kernel<T>), dim3(p.embed_blocks + p.copy_blocks), dim3(256), 0, st.stream,
                                       p);
                    if (!hip_ok(hipGetLastError(), "layout launch")) return 2;
                }
                if (kept) xb = const_cast<uint4 *>(kept);
                st.last_conv_resident = 1;
                return conv_halo_wg_launch(d, xb, gb, gstride, ws, dW, Hp, Wp, S0, S1);
            }
        }
    }
    if constexpr (ES == 2) {
        // 3x3 "same" channel-minor layers: the same kernel on the caller's tensors in place
        if (hwc && conv_halo_wg_hwc_fits(d, X, dY) &&
            (st.gemm_path == 5 || (st.gemm_path == 0 && conv_halo_wg_hwc_preferred(d)))) {
            int S0 = 1, S1 = 1;
            const size_t ws_bytes = conv_halo_wg_partial_bytes(d, d.Hin + 1, d.Win + 1, &S0, &S1);
            if (ws_bytes <= ((size_t)1 << 30)) {
                float *ws = workspace(ws_bytes);
                if (!ws) return 2;
                st.last_conv_resident = 1;
                return conv_halo_wg_hwc_launch(d, X, dY, ws, dW, S0, S1);
            }
        }
    }
    if (hwc) {  // channel-minor: both operands are [position][channel] matrices read 16 bytes along the channels
        if (d.Cout % VEC || reinterpret_cast<uintptr_t>(X) % 16 || reinterpret_cast<uintptr_t>(dY) % 16) return -1;
        // (no direct kernel for this layout: the alternative is the gathering GEMM, which this route beats from 64
        // channels on and a few hundred positions (measured 11.3 against 7.8 us for one 64-channel 8x8 sample,
        // 11.8 against 13.3 us for eight)
        // and about 2e8 multiply-adds per tap: a sweep over 64..512 channels on 7x7..56x56 images at batch 8..128 has
        // the gathering GEMM ahead below that, e.g. 13.0 against 16.3 us for 64 -> 64 on 28x28 at batch 8 and 23.7
        // against 34.1 us for 256 -> 256 on 14x14 at batch 8, and this route ahead above, 28.3 against 40.7 us for
        // 64 -> 128 on 28x28 at batch 32, 41.7 against 69.4 us for 256 -> 256 on 14x14 at batch 32)
        if (st.gemm_path != 3 &&
            (d.Cin < 64 || d.Cout < 64 || (double)d.batch * d.Ho * d.Wo * d.Cin * d.Cout < 2e8))
            return -1;
    } else {
        if (d.x_sy != d.Win) return -1;
        if (st.gemm_path != 3 && (d.Cin < 128 || d.Cout < 128)) return -1;  // measured: below that the direct kernel wins
        // (and below about 8000 padded positions the gathering GEMM does: 12 against 29 us for eight 256 -> 256 7x7
        // samples, 25 against 27 us for 128 -> 128 on 14x14 at batch 32)
        if (st.gemm_path != 3 && (long long)d.batch * (d.Hin + 2) * (d.Win + 2) < 8192)
            return -1;
    }
    if (st.gemm_path == 2) return -1;
    const int taps = d.KH * d.KW;
    int Hp, Wp;
    conv_padded_grid(d, &Hp, &Wp);
    if (!conv_output_fits_pads(d)) return -1;
    const int cblocks = d.Cin / VEC;
    const long long plane = (long long)Hp * Wp * VEC;
    const long long Kp = (long long)d.batch * Hp * Wp;              // padded positions of all samples
    const long long Kr = (Kp + SK - 1) / SK * SK;
    const long long margin = (Kr - Kp) + (long long)(d.KH - 1) * Wp + d.KW + SK;  // positions read past the end
    // (channel-major: the planes of a channel block follow each other, so only the last one needs the margin;
    // channel-minor: a position is cblocks chunks)
    const long long xb_chunks = hwc ? (long long)cblocks * ((long long)d.batch * Hp * Wp + margin)
                                    : (long long)cblocks * d.batch * Hp * Wp + margin;
    const long long gy_elems = (long long)d.Cout * Kr;
    if (xb_chunks * 16 >= ((long long)1 << 31) || gy_elems * ES >= ((long long)1 << 31) || Kr >= ((long long)1 << 31))
        return -1;
    // fp16 layers whose channel counts fill 256x256 tiles take those (a quarter less LDS traffic and half the L2 -> LDS
    // traffic per MFMA of the 128x128 tile, and a quarter of the partial sums)
    const int bm = (ES == 2 && d.Cout % 256 == 0 && d.Cin % 256 == 0 && st.gemm_path != 4) ? 256
                   : (d.Cout >= 128 && d.Cin >= 128)                                          ? 128
                                                                                              : 64;
    const long long tiles = (long long)((d.Cout + bm - 1) / bm) * ((d.Cin + bm - 1) / bm);
    // k splits: one workgroup of this tile holds a CU (96 KB of ring), so the launch runs in rounds of num_cu
    // workgroups.  Take the split count with the least rounds x (slabs per workgroup + the fixed cost of a
    // workgroup's prologue and fp32 partial-sum epilogue, about six slabs' worth).
    const long long max_s = Kr / (4 * SK) > 0 ? Kr / (4 * SK) : 1;
    const long long slabs = Kr / SK, fixed = 6;
    long long S = 1, best = -1;
    const long long slots = (long long)st.num_cu * (bm == 64 ? 2 : 1);  // two workgroups of the small tile share a CU
    for (long long s = 1; s <= max_s && s * tiles * taps <= 8 * slots; ++s) {
        const long long rounds = (s * tiles * taps + slots - 1) / slots;
        const long long cost = rounds * ((slabs + s - 1) / s + fixed);
        if (best < 0 || cost < best) {
            best = cost;
            S = s;
        }
    }
    long long kchunk = ((Kr + S - 1) / S + SK - 1) / SK * SK;
    S = (Kr + kchunk - 1) / kchunk;
    const size_t ws_bytes = (size_t)taps * S * d.Cout * d.Cin * sizeof(float);
    if (ws_bytes > ((size_t)1 << 30)) return -1;
    char *buf = static_cast<char *>(scratch((size_t)xb_chunks * 16 + 256 + (size_t)gy_elems * ES));
    if (!buf) return 2;
    uint4 *xb = reinterpret_cast<uint4 *>(buf);
    T *gy = reinterpret_cast<T *>(buf + (((size_t)xb_chunks * 16 + 255) & ~(size_t)255));
    float *ws = workspace(ws_bytes);
    if (!ws) return 2;
    const long long cb_stride = (long long)d.batch * plane;
    if (cb_stride >= ((long long)1 << 31)) return -1;
    if (!hwc) {
        if (int rc = blocked_padded_copy<T>(reinterpret_cast<const T *>(X), xb, d, Hp, Wp, margin)) return rc;
        hipLaunchKernelGGL((embed_gradient_kernel<T>), dim3((unsigned)((gy_elems / VEC + 255) / 256)), dim3(256), 0,
                           st.stream, reinterpret_cast<const T *>(dY), reinterpret_cast<uint4 *>(gy), d.batch, d.Cout,
                           d.Ho, d.Wo, Hp, Wp, Kr, gy_elems / VEC);
    } else {
        hipLaunchKernelGGL(hwc_to_padded_kernel, dim3((unsigned)((xb_chunks + 255) / 256)), dim3(256), 0, st.stream,
                           reinterpret_cast<const uint4 *>(X), xb, d.batch, d.Hin, d.Win, Hp, Wp, d.padU, d.padL, cblocks,
                           xb_chunks);
        if (!hip_ok(hipGetLastError(), "padded copy launch")) return 2;
        hipLaunchKernelGGL(embed_gradient_hwc_kernel, dim3((unsigned)((gy_elems / VEC + 255) / 256)), dim3(256), 0,
                           st.stream, reinterpret_cast<const uint4 *>(dY), reinterpret_cast<uint4 *>(gy), d.batch,
                           d.Cout / VEC, d.Ho, d.Wo, Hp, Wp, gy_elems / VEC);
    }
    if (!hip_ok(hipGetLastError(), "gradient layout launch")) return 2;

    GemmArgs q = {};
    q.A = gy;
    q.B = xb;
    q.C = dW;
    q.ws = ws;
    q.N = d.Cout;
    q.M = d.Cin;
    q.K = (int)Kr;
    q.a.HL = q.a.WL = q.b.HL = q.b.WL = 1;
    if (!hwc) {
        q.a.row = axis_plain(d.Cout, (int)Kr);
        q.a.k = axis_plain((int)Kr, 1);
        q.a.mode = FILL_VEC_K;
        q.b.row = axis_two(d.Cin, VEC, (int)cb_stride, 1);
        q.b.k = axis_plain((int)Kr, VEC);
        q.c.n = axis_plain(d.Cout, d.Cin * taps);
        q.c.m = axis_plain(d.Cin, taps);
    } else {
        q.a.row = axis_plain(d.Cout, 1);
        q.a.k = axis_plain((int)Kr, d.Cout);
        q.a.mode = FILL_VEC_R;
        q.b.row = axis_plain(d.Cin, 1);
        q.b.k = axis_plain((int)Kr, d.Cin);
        q.c.n = axis_plain(d.Cout, d.Cin * taps);
        q.c.m = axis_plain(d.Cin, 1);
    }
    q.b.mode = FILL_VEC_R;
    q.kchunk = (int)kchunk;
    q.splits = (int)(taps * S);
    q.tap_splits = (int)S;
    q.tap_kw = d.KW;
    q.tap_jump_x = (long long)(hwc ? d.Cin : VEC) * ES;  // one padded position further in the second operand
    q.tap_jump_y = (long long)Wp * (hwc ? d.Cin : VEC) * ES;
    if (!plain_operand<T>(q.a, q.kchunk, q.K) || !plain_operand<T>(q.b, q.kchunk, q.K)) return -1;
    int rc;
    if constexpr (ES == 2) {
        rc = bm == 256   ? launch_plain<T, 256, 256, 512, 2, 4, 1, 2, 1>(q, st.stream)
             : bm == 128 ? launch_plain<T, 128, 128, 512, 2, 2, 2, 3, 1>(q, st.stream)
                         : launch_plain<T, 64, 64, 1024, 2, 2, 4, 3, 1>(q, st.stream);
    } else {
        rc = bm == 128 ? launch_plain<T, 128, 128, 512, 2, 2, 2, 3, 1>(q, st.stream)
                       : launch_plain<T, 64, 64, 1024, 2, 2, 4, 3, 1>(q, st.stream);
    }
    if (rc != 0 || q.splits == 1) return rc;  // a single 1x1 tap without k split wrote dW itself
    const long long total = (long long)d.Cout * d.Cin;
    hipLaunchKernelGGL((taps_wg_reduce_kernel<T>), dim3((unsigned)((total + 63) / 64), taps), dim3(256), 0, st.stream,
                       ws, reinterpret_cast<T *>(dW), total, (int)S, taps, d.Cin, hwc ? 1 : 0);
    return hip_ok(hipGetLastError(), "tap reduce launch") ? 0 : 2;
}

// Backward pass of a 3x3 "same" layer (pads of both sides add up to 2, unit stride, fp16, channel-major): the weight
// gradient and the input gradient read the SAME channel-blocked copy of the output gradient - the input gradient
// as its padded input (the gradient sits KH-1-padU rows / KW-1-padL columns inside each grid), the weight gradient
// that many positions further on as the gradient embedded at the top left of the grid.  One layout pass less than
// the two calls on their own.
template <typename T>
int conv_halo_bw(const ConvTileDesc &fwd, const ConvTileDesc &ig, const void *X, const void *dY, const void *Wt,
                 void *dW, void *dX) {
    if constexpr (sizeof(T) != 2) {
        return -1;
    } else {
        State &st = state();
        constexpr int VEC = 8;
        int Hp, Wp, Hpi, Wpi;
        conv_padded_grid(fwd, &Hp, &Wp);
        conv_padded_grid(ig, &Hpi, &Wpi);
        if (Hp != Hpi || Wp != Wpi || fwd.x_sy != fwd.Win || ig.x_sy != ig.Win) return -1;
        if (!conv_halo_fits(ig, Hp, Wp) || !conv_halo_wg_fits(fwd, Hp, Wp) || !conv_halo_wg_preferred(fwd)) return -1;
        if (!(st.gemm_path == 0 || st.gemm_path == 5)) return -1;
        // The input gradient's persistent kernel needs enough tiles (256 positions x 128 filters): with fewer than
        // about 40 the two single steps, whose input gradient then goes another way, are faster than the pair
        // (in turns in one process, pair against two calls: 128 -> 128 on 28x28 at batch 8, 27 tiles, 40.4 / 36.8 us;
        // 512 -> 512 on 14x14 at batch 8, 32 tiles, 91.5 / 73.7; 256 -> 256 on 32x32 at batch 4, 36 tiles, 55.0 / 46.5;
        // 128 -> 128 on 28x28 at batch 12, 40 tiles, 41.1 / 44.9; 256 -> 256 on 14x14 at batch 24, 44 tiles, 57.9 / 62.6).
        const long long ig_tiles = ((long long)ig.batch * Hp * Wp + 255) / 256 * ((ig.Cout + 127) / 128);
        if (st.gemm_path == 0 && ig_tiles < 40) return -1;
        const long long P = (long long)fwd.batch * Hp * Wp;
        const int goff = ig.padU * Wp + ig.padL;  // where the weight gradient's view of the copy starts
        const long long gstride = conv_halo_wg_gradient_stride(fwd, Hp, Wp) + 128;
        if (goff > 128) return -1;
        const long long xmargin = conv_halo_wg_margin(), gmargin = conv_halo_margin() + 128;
        const long long xb_chunks = (long long)(fwd.Cin / VEC) * P + xmargin;
        const long long gb_chunks = (long long)(fwd.Cout / VEC) * gstride + gmargin;
        const long long wr_elems = (long long)ig.Cout * 9 * ig.Cin;
        int S0 = 1, S1 = 1;
        const size_t ws_bytes = conv_halo_wg_partial_bytes(fwd, Hp, Wp, &S0, &S1);
        if (xb_chunks * 16 >= ((long long)1 << 31) || gb_chunks * 16 >= ((long long)1 << 31) ||
            ws_bytes > ((size_t)1 << 30))
            return -1;
        char *buf = static_cast<char *>(scratch((size_t)(xb_chunks + gb_chunks) * 16 + (size_t)wr_elems * 2 + 768));
        if (!buf) return 2;
        float *ws = workspace(ws_bytes);
        if (!ws) return 2;
        uint4 *xb = reinterpret_cast<uint4 *>(buf);
        char *gb = buf + (((size_t)xb_chunks * 16 + 255) & ~(size_t)255);
        T *wr = reinterpret_cast<T *>(gb + (((size_t)gb_chunks * 16 + 255) & ~(size_t)255));
        // One launch for the layout passes, all independent of each other: the shared copy of the output gradient, the
        // zero margin behind its last block (the input-gradient kernel reads past the end), the blocked copy of the
        // input unless the call was handed one, the flipped, transposed filters of the input gradient.
        const uint4 *kept = cached_input(fwd, Hp, Wp, xb_chunks);
        {
            const long long Pg = (long long)ig.batch * Hp * Wp, e_chunks = (long long)(ig.Cin / VEC) * gstride;
            if (e_chunks >= ((long long)1 << 31) || gstride < Pg) return -1;
            TapPrepArgs p = {};
            p.e_in = dY;
            p.e_out = reinterpret_cast<uint4 *>(gb);
            p.e_Ho = ig.Hin; p.e_Wo = ig.Win; p.e_Hp = Hp; p.e_Wp = Wp; p.e_pu = ig.padU; p.e_pl = ig.padL;
            p.e_sb = (long long)ig.Cin * ig.Hin * ig.Win;
            p.e_sc = (long long)ig.Hin * ig.Win;
            p.e_P = (unsigned)Pg;
            p.e_pstride = (unsigned)gstride;
            p.e_total = (unsigned)e_chunks;
            p.embed_blocks = (unsigned)((e_chunks + 255) / 256);
            p.zero_at = reinterpret_cast<uint4 *>(gb) + (long long)(fwd.Cout / VEC) * gstride;
            p.zero_n = (unsigned)gmargin;
            p.zero_blocks = (unsigned)((gmargin + 255) / 256);
            if (!kept) {
                const int cblocks = fwd.Cin / VEC;
                p.in = X;
                p.xb = xb;
                p.B = fwd.batch; p.H = fwd.Hin; p.W = fwd.Win; p.Hp = Hp; p.Wp = Wp; p.padU = fwd.padU; p.padL = fwd.padL;
                p.cblocks = cblocks;
                p.sb = fwd.x_sb; p.sc = fwd.x_sc;
                p.xb_total = (long long)cblocks * fwd.batch * Hp * Wp + xmargin;
                p.copy_blocks = (unsigned)((p.xb_total + 255) / 256);
            }
            p.w = Wt;
            p.wr = wr;
            p.C = ig.Cin; p.KW = 3; p.taps = 9;
            p.w_base = ig.w_base; p.w_sm = ig.w_sm; p.w_sc = ig.w_sc; p.w_sy = ig.w_sy; p.w_sx = ig.w_sx;
            p.wr_total = wr_elems;
            const unsigned long long blocks = (unsigned long long)p.embed_blocks + p.zero_blocks + p.copy_blocks +
                                              (unsigned long long)((wr_elems + 255) / 256);
            if (blocks >= (1ull << 31)) return -1;
            hipLaunchKernelGGL((tap_prepare_kernel<T>), dim3((unsigned)blocks), dim3(256), 0, st.stream, p);
            if (!hip_ok(hipGetLastError(), "layout launch")) return 2;
        }
        if (kept) xb = const_cast<uint4 *>(kept);
        st.last_conv_resident = 1;
        if (int rc = conv_halo_wg_launch(fwd, xb, gb + (size_t)goff * 16, gstride, ws, dW, Hp, Wp, S0, S1)) return rc;
        return conv_halo_launch(ig, gb, wr, dX, Hp, Wp, gstride);
    }
}
template int conv_halo_bw<float>(const ConvTileDesc &, const ConvTileDesc &, const void *, const void *, const void *,
                                 void *, void *);
template int conv_halo_bw<half_t>(const ConvTileDesc &, const ConvTileDesc &, const void *, const void *, const void *,
                                  void *, void *);

template int conv_taps_wg<float>(const ConvTileDesc &, const void *, const void *, void *);
template int conv_taps_wg<half_t>(const ConvTileDesc &, const void *, const void *, void *);

template int conv_taps<float>(const ConvTileDesc &, const void *, const void *, void *, const OutMap &);
template int conv_taps<half_t>(const ConvTileDesc &, const void *, const void *, void *, const OutMap &);

}  // namespace ptl
