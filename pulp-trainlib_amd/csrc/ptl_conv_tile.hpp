// Direct (raw-tile) convolution for channel-major tensors: host interface.
#pragma once
#include "ptl_common.hpp"

struct ptl_conv_cache;
struct ptl_wg_batch;
struct ptl_norm_stats;
struct ptl_grad_post;

namespace ptl {

// out(b, m, y, x) = sum_{ci, ky, kx} in(b, ci, y*sh + ky - padU, x*sw + kx - padL) * w(m, ci, ky, kx)
// with in() zero outside the image, in(b, ci, iy, ix) at X[b*x_sb + ci*x_sc + iy*x_sy + ix] and
// w(m, ci, ky, kx) at Wt[w_base + m*w_sm + ci*w_sc + ky*w_sy + kx*w_sx].
struct ConvTileDesc {
    int batch, Cin, Hin, Win;
    int Cout, Ho, Wo;
    int KH, KW, sh, sw;
    int padU, padD, padL, padR;
    long long x_sb, x_sc;
    int x_sy;
    int w_base, w_sm, w_sc, w_sy, w_sx;
    // 1: the input is channel-minor, in(b, ci, iy, ix) at X[((b*Hin + iy)*Win + ix)*Cin + ci] (x_s* unused);
    // with Cin a multiple of the 16-byte vector it already consists of the chunks the kernel wants
    int in_hwc;
    // 2: the convolution reads the input zero-stuffed by two (element (y, x) of the tensor at (2y, 2x) of a
    // (2*Hin - 1) x (2*Win - 1) image, zeros between): the input gradient of a stride-2 layer as a unit-stride pass
    // over its output gradient.  Only the small-layer kernel takes it; 0 or 1: the tensor as it is.
    int in_dil;
};

// Launches the direct kernel; the output is written through `c` (n = pixel index over
// (sample, row, column), m = filter).  Returns 0, a positive status on a HIP error, or -1
// when the geometry does not fit the kernel (the caller then takes the GEMM route).
template <typename T>
int conv_tile(const ConvTileDesc &d, const void *X, const void *Wt, void *Y, const OutMap &c);

// 3x3 layers with at most 64 channels on either side, dense channel-major tensors: one launch that reads the
// caller's tensors directly (ptl_conv_small.hip).  Y is the dense channel-major output [batch][Cout][Ho][Wo].
// Returns -1 when the layer does not fit or is large enough for the persistent kernels to be ahead.
template <typename T>
int conv_small(const ConvTileDesc &d, const void *X, const void *Wt, void *Y);
// Weight gradient of such a layer (unit stride, output as wide as the input), and weight + input gradient with the
// two products in one launch (`fwd` describes the forward layer, `ig` the input gradient as a forward pass over dY).
// (`may_defer`: dW is the caller's own device tensor, so its sums may wait in a batch given with conv_small_defer_to)
template <typename T>
int conv_small_wg(const ConvTileDesc &d, const void *X, const void *dY, void *dW, bool may_defer);
template <typename T>
int conv_small_bw(const ConvTileDesc &fwd, const ConvTileDesc &ig, const void *X, const void *dY, const void *Wt,
                  void *dW, void *dX, bool may_defer);

}  // namespace ptl

namespace ptl {

// Quotients by a divisor fixed per launch: magic = ceil(2^32 / d) gives exact n / d for
// n, d < 2^16; magic 0 stands for d == 1.
inline unsigned magic_of(int dv) { return dv <= 1 ? 0u : (unsigned)((((unsigned long long)1 << 32) + dv - 1) / dv); }
#if defined(__HIPCC__)
__device__ inline int fast_div(int n, unsigned magic) { return magic ? (int)__umulhi((unsigned)n, magic) : n; }
#endif

// Raw input rows (counted over padded images laid end to end) that a tile of `bm` consecutive
// output pixels touches, maximised over all tiles: exact, from one period of the tile / image
// pattern, remembered for the last geometry asked.
inline int conv_raw_rows(int bm, int Ho, int Wo, int sh, int KH, int THP, long long npix) {
    static int key[6] = {0, 0, 0, 0, 0, 0}, val = 0;
    static long long key_n = 0;
    if (key[0] == bm && key[1] == Ho && key[2] == Wo && key[3] == sh && key[4] == KH && key[5] == THP && key_n == npix)
        return val;
    const long long PP = (long long)Ho * Wo;
    long long a = PP, b = bm;
    while (b) {
        long long t = a % b;
        a = b;
        b = t;
    }
    long long period_tiles = PP / a;  // tiles until the (tile start mod image) pattern repeats
    const long long tiles = (npix + bm - 1) / bm;
    if (period_tiles > tiles) period_tiles = tiles;
    int best = 0;
    for (long long t = 0; t < period_tiles; ++t) {
        const long long p0 = t * bm, p1 = (p0 + bm - 1 < npix - 1) ? p0 + bm - 1 : npix - 1;
        const long long g0 = (p0 / PP) * THP + ((p0 % PP) / Wo) * sh, g1 = (p1 / PP) * THP + ((p1 % PP) / Wo) * sh;
        if ((int)(g1 - g0) > best) best = (int)(g1 - g0);
    }
    // the last tile of the tensor may be cut short; it never needs more than a full one
    val = best + KH;
    key[0] = bm; key[1] = Ho; key[2] = Wo; key[3] = sh; key[4] = KH; key[5] = THP;
    key_n = npix;
    return val;
}

// Weight gradient of the same convolution:
//   dW(co, ci, ky, kx) = sum_{b, y, x} dY(b, co, y, x) * in(b, ci, y*sh + ky - padU, x*sw + kx - padL)
// with dY channel-major [b][Cout][Ho*Wo] and dW dense [Cout][Cin][KH][KW].  Returns 0, a positive
// status on a HIP error, or -1 when the geometry does not fit the kernel.
// The same convolution as a sum over filter taps on the look-up-free GEMM (unit stride, channel-major input,
// channels a multiple of a slab); -1 when the geometry does not fit.  Input and filters are re-laid in scratch.
template <typename T>
int conv_taps(const ConvTileDesc &d, const void *X, const void *Wt, void *Y, const OutMap &c);

// The padded grid of the tap-sum and resident-tile routes: every sample takes Hin + max(padU, padD) rows of
// Win + max(padL, padR) positions, the tensor padU rows / padL columns inside it.  The zero rows above a sample are
// also the zero rows below the one before it, the zero columns left of a row the ones right of the row before it
// (a window that runs off a row's end continues at the start of the next row), so a 3x3 "same" layer pads by ONE
// row and ONE column per sample instead of two: fewer bytes to write and read, and fewer positions that the
// kernels compute and drop.  Behind the last sample of a channel block the next block's first rows (or the
// margin behind the last block) are the zeros.
inline void conv_padded_grid(const ConvTileDesc &d, int *Hp, int *Wp) {
    *Hp = d.Hin + (d.padU > d.padD ? d.padU : d.padD);
    *Wp = d.Win + (d.padL > d.padR ? d.padL : d.padR);
}
// whether the output is the "valid" convolution of the fully padded input (what these routes compute)
inline bool conv_output_fits_pads(const ConvTileDesc &d) {
    return d.Ho == d.Hin + d.padU + d.padD - d.KH + 1 && d.Wo == d.Win + d.padL + d.padR - d.KW + 1;
}

// 3x3 unit-stride fp16 channel-major layers with the input tile resident in LDS for all taps (same prepared
// operands as the tap-sum route: blocked padded input with conv_halo_margin() readable chunks behind it, tap-major
// filters).  Y is the dense channel-major output [batch][Cout][Ho][Wo].
bool conv_halo_fits(const ConvTileDesc &d, int Hp, int Wp);
long long conv_halo_margin();
// Chunk i of gb[cb][p], p < pstride: the tensor element t[b][8 cb .. + 7][yp - pu][xp - pl] at p = (b, yp, xp) of the
// padded grid, zero outside the tensor and from the last padded position on (the blocked copy of an output gradient
// that the resident-tile weight- and input-gradient kernels read).
__device__ inline void halo_embed_chunk(unsigned i, const half_t *__restrict__ dy, uint4 *__restrict__ out, int Ho,
                                        int Wo, int Hp, int Wp, int pu, int pl, long long sb, long long sc, unsigned P,
                                        unsigned pstride) {
    const unsigned cb = i / pstride, p = i - cb * pstride;
    union {
        uint4 v;
        half_t e[8];
    } u;
    u.v = make_uint4(0, 0, 0, 0);
    if (p < P) {
        const unsigned r = p / (unsigned)Wp, xp = p - r * (unsigned)Wp;
        const unsigned b = r / (unsigned)Hp, yy = r - b * (unsigned)Hp - (unsigned)pu, xx = xp - (unsigned)pl;
        if (yy < (unsigned)Ho && xx < (unsigned)Wo) {
            const half_t *src = dy + b * sb + (long long)(cb * 8) * sc + (long long)yy * Wo + xx;
#pragma unroll
            for (int e = 0; e < 8; ++e) u.e[e] = src[e * sc];
        }
    }
    out[i] = u.v;
}

// A second copy of the output for the layer that reads it next: channel-blocked and padded for THAT layer,
// [channels / 8][batch][Hp][Wp] 16-byte chunks with the output pixel (y, x) at (y + padU, x + padL); the kernel
// writes the pixels, the halo is the caller's (zero) business.
struct HaloOutCopy {
    void *buf;
    int Hp, Wp, padU, padL;
    int relu;  // 1: the copy holds max(output, 0)
};
int conv_halo_launch(const ConvTileDesc &d, const void *xb, const void *wr, void *Y, int Hp, int Wp,
                     long long pstride = 0, const HaloOutCopy *out_copy = nullptr);  // pstride: positions between channel blocks of xb (0: batch*Hp*Wp)
// The same layers with channel-minor tensors read in place (X [batch][H][W][Cin], tap-major filters, Y
// [batch][H][W][Cout]): one launch, the zero border comes from the addresses of the loads.
bool conv_halo_hwc_fits(const ConvTileDesc &d, const void *X, const void *Y);
int conv_halo_hwc_launch(const ConvTileDesc &d, const void *X, const void *wr, void *Y);
int conv_halo_embed(const void *t, void *out, int batch, int C, int Hs, int Ws, int Hp, int Wp, int pu, int pl,
                    long long pstride);

// Weight gradient of the same layers on the same layouts (gradient embedded in the padded grid, channel-blocked):
// partial sums per tap and position split + one reduction.  See ptl_conv_halo.hip for the buffer sizes.
bool conv_halo_wg_fits(const ConvTileDesc &d, int Hp, int Wp);
bool conv_halo_wg_preferred(const ConvTileDesc &d);  // fits, and measured faster than the other weight-gradient routes
long long conv_halo_wg_margin();
long long conv_halo_wg_gradient_stride(const ConvTileDesc &d, int Hp, int Wp);
size_t conv_halo_wg_partial_bytes(const ConvTileDesc &d, int Hp, int Wp, int *S0, int *S1);
// The same kernel on channel-minor tensors read in place (3x3 "same" layers, Cout a multiple of 128): one launch + the
// addition of the partial sums; ws sized by conv_halo_wg_partial_bytes() for Hp = Hin + 1, Wp = Win + 1.
bool conv_halo_wg_hwc_fits(const ConvTileDesc &d, const void *X, const void *dY);
bool conv_halo_wg_hwc_preferred(const ConvTileDesc &d);
int conv_halo_wg_hwc_launch(const ConvTileDesc &d, const void *X, const void *dY, float *ws, void *dW, int S0, int S1);
int conv_halo_wg_launch(const ConvTileDesc &d, const void *xb, const void *gb, long long gstride, float *ws, void *dW,
                        int Hp, int Wp, int S0, int S1);

// Weight gradient and input gradient of one 3x3 "same" layer sharing one blocked copy of the output gradient;
// -1 when the layer does not fit both resident-tile kernels.
template <typename T>
int conv_halo_bw(const ConvTileDesc &fwd, const ConvTileDesc &ig, const void *X, const void *dY, const void *Wt,
                 void *dW, void *dX);

// The caller-owned copy of a layer's blocked, padded input (struct ptl_conv_cache) for the call in progress: `fill` is
// written by the forward route that builds such a copy, `use` read by the weight-gradient routes.  Both null outside
// the *_cached entry points.
void conv_cache_set(struct ::ptl_conv_cache *fill, const struct ::ptl_conv_cache *use);
// Layers in a row (the *_chained forward entry point): `in` is a copy of this layer's input that the forward route
// may read instead of making one (valid: left there by the layer before), `out` a prepared buffer for the copy of
// this layer's output that the next layer reads.  Both null outside that entry point.
void conv_cache_chain(const struct ::ptl_conv_cache *in, struct ::ptl_conv_cache *out);
// Where the small-layer weight gradient leaves its partial sums instead of adding them up itself (nullptr: nowhere);
// the one launch that adds up all the layers a batch holds.
void conv_small_defer_to(struct ::ptl_wg_batch *batch);
template <typename T>
int conv_small_flush(struct ::ptl_wg_batch *batch);
// Where the small-layer forward kernel leaves per-workgroup sums of its output and of its squares per filter (struct
// ptl_norm_stats; nullptr: nowhere).  The call marks the struct valid when it filled it.
void conv_small_stats_to(struct ::ptl_norm_stats *st);
// A normalisation layer that the next forward call of the small-layer kernel applies while it loads its input
// (nullptr: none).  x: the normalisation's input; out: its output = the convolution's input tensor, written by the
// call; skip: added after the normalisation (or null); weight, bias, eps: the layer's; part / parts / count: the
// sums of x ([channel][part][4] floats).  A call that cannot honour it launches nothing and returns CONV_PRE_REFUSED;
// conv_small_pre_pending() tells a caller that routes elsewhere that it must not.
struct ConvPreNorm {
    const void *x, *skip, *weight, *bias, *eps;
    void *out;
    const float *part;
    int parts, relu;
    size_t count;
};
constexpr int CONV_PRE_REFUSED = -3;
void conv_small_pre_to(const ConvPreNorm *pre);
bool conv_small_pre_pending();
// Room in a batch of deferred weight-gradient sums for another layer's partial sums (`parts` of them, `part_elems`
// floats each, in the order the flush reads: [part][32-channel block][tap][filter row][channel of the block]) that
// the flush will add up into dW[filter][channel][tap]; nullptr when the batch cannot take it.
float *wg_batch_reserve(struct ::ptl_wg_batch *b, void *dW, int parts, int filters, int channels, int taps);
// What the input gradient of the next one-call backward does in its epilogue (struct ptl_grad_post) and where the sums
// of the gradient it forms go; sums->valid tells whether it did.  Cleared with (nullptr, nullptr).
void conv_small_post_to(const struct ::ptl_grad_post *post, struct ::ptl_norm_stats *sums);

// Weight gradient over filter taps on the same GEMM (partial sums per tap and k split + one reduction).
template <typename T>
int conv_taps_wg(const ConvTileDesc &d, const void *X, const void *dY, void *dW);

template <typename T>
int conv_tile_wg(const ConvTileDesc &d, const void *X, const void *dY, void *dW);

}  // namespace ptl
