// Direct convolution on MFMA for channel-major (CHW) tensors: forward, and input
// gradient as a forward pass over the (zero-stuffed) output gradient with flipped,
// transposed filters.
//
// The GEMM route fetches every element of the implicit im2col matrix from global
// memory, Hk*Wk times per input element and one lane-load each.  Here a workgroup
// owns BM consecutive output pixels (raster order over sample, row, column) and BN
// output channels, and
//   * gets the input rows those pixels touch ONCE into LDS, as [channel block][row][col]
//     chunks of 16 bytes that hold VEC consecutive channels of one input position, the
//     padding halo as zeros (raw tile).  Where input rows are whole aligned 16-byte groups
//     (the usual case) the rows come in pixel-major by LDS-DMA straight from the tensor into
//     a staging buffer and are re-laid LDS to LDS; otherwise a first kernel re-lays the whole
//     input in exactly these chunks ([sample][channel block][row][col]) and the raw tile is
//     filled by LDS-DMA from that copy (halo chunks read a zero buffer);
//   * loads its BN filters into LDS as [filter][tap][channel] (rows padded to an odd
//     multiple of 16 bytes, which spreads sixteen consecutive filters over all 64 banks),
//     once per workgroup: a workgroup then walks several pixel tiles;
//   * runs the contraction tap by tap, channel blocks innermost: the A fragment of a lane
//     (one pixel, VEC channels) is ONE ds_read_b128 at rawoff(pixel) + tapoff(hk, wk), the
//     B fragment another, i.e. the im2col matrix never exists, not even in LDS;
//   * stores straight from the accumulators: filters are the MFMA rows and pixels the
//     columns, so the 32 lanes of a half-wave write 32 consecutive pixels of one filter.
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
    const void *zero;  // at least 16 readable zero bytes
    int fast_pix;      // 1: pixel coordinates by reciprocal multiplication (tile-relative quotients below 2^16)
    int nfast;         // 1: the output's pixel axis is (sample, pixel-in-sample) with the sample size as radix
    unsigned magic_pp, magic_wo, magic_thp;
    int in_sb, in_scb, in_sy, in_sx;  // chunk strides of the chunked input: sample, channel block, row, column
    int in_cblocks;    // channel blocks that exist in it (the rest of CinP is zeros)
    int m_unit;        // 1: consecutive filters are consecutive output elements (4-element stores)
    int raw_chunks;    // chunks of one raw slab (two channel blocks) rounded up to whole waves
    int stage_chunks;  // chunks of one staging slab (KSTEP channels x RR rows x whole input rows), whole waves
    int xg;            // 16-byte groups per input row
    unsigned magic_xg, magic_rrxg;
    unsigned magic_tw, magic_rr, magic_perm, magic_cb, magic_kw;  // ceil(2^32 / d): exact for n, d < 2^16
    int c_mode;
};


template <typename T, int BM, int BN, bool STAGED>
__global__ __launch_bounds__((BM / 32) * 64) void conv_tile_kernel(const ConvTileArgs a) {
    constexpr int NT = (BM / 32) * 64;
    constexpr int ES = (int)sizeof(T), VEC = 16 / ES, KSTEP = 2 * VEC, FN = BN / 32;
    extern __shared__ __attribute__((aligned(16))) char smem[];
    char *bl = smem;                                          // filters [BN][b_pitch]
    // raw slab(s) [channel block][row][col] of VEC channels: two when they are filled from the
    // blocked copy of the input, one when they are built from the staging buffers that follow
    uint4 *raw = reinterpret_cast<uint4 *>(smem + a.b_bytes);
    T *stage = reinterpret_cast<T *>(raw + a.raw_chunks);  // STAGED: two pixel-major slabs [channel][row][col]
    __shared__ int mlut[BN];      // per filter: output offset

    const ConvTileDesc &d = a.d;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave;
    const int m0 = blockIdx.y * BN;
    const int PP = d.Ho * d.Wo;
    const uint4 *__restrict__ Xb = reinterpret_cast<const uint4 *>(a.X);  // blocked input (not STAGED)
    const T *__restrict__ X = reinterpret_cast<const T *>(a.X);           // channel-major input (STAGED)
    const T *__restrict__ Wt = reinterpret_cast<const T *>(a.Wt);
    const int kg = lane >> 5, lr = lane & 31;
    const int cblocks = a.CinP / VEC;

    // Software pipeline over the workgroup's slabs.  A slab is one pixel tile times one k step
    // of channels (two channel blocks, all taps); a tile's slabs accumulate into the same
    // registers.  The LDS-DMA of the next slab is enqueued into the other raw buffer before the
    // current one is computed, so its latency hides behind the MFMAs and stores; one barrier per
    // slab (it has landed for every wave, and every wave is done with the previous one, whose
    // buffer is refilled next).  Nothing crosses threads except the raw tile itself: each lane
    // derives its own addresses.
    const unsigned raw_lds = (unsigned)(uintptr_t)(lds_char *)raw;
    const unsigned stage_lds = (unsigned)(uintptr_t)(lds_char *)stage;
    auto enqueue = [&](int tile, int cs, int buf) {
        const int n0 = tile * BM;
        const int b0 = n0 / PP, y0 = (n0 - b0 * PP) / d.Wo;
        const int t0 = y0 * d.sh;  // first raw row, counted inside the padded image of sample b0
        if (STAGED) {
            // pixel-major staging slab straight from the tensor: chunk c = (channel * RR + row) * XG + group of
            // VEC columns; rows outside the image and channels beyond the tensor read the zero buffer
            const int rrxg = a.RR * a.xg;
            for (int c0 = wave * 64; c0 < a.stage_chunks; c0 += NT) {
                const int c = c0 + lane;
                const int ch = fast_div(c, a.magic_rrxg), r = c - ch * rrxg;
                const int rr = fast_div(r, a.magic_xg), xg = r - rr * a.xg;
                const int t = t0 + rr, db = fast_div(t, a.magic_thp);
                const int b = b0 + db, iy = t - db * a.THP - d.padU, chn = cs * KSTEP + ch;
                const bool ok = ch < KSTEP && chn < d.Cin && b < d.batch && iy >= 0 && iy < d.Hin;
                const int idx = b * (int)d.x_sb + chn * (int)d.x_sc + iy * d.Win + xg * VEC;
                const char *src = ok ? reinterpret_cast<const char *>(X + idx) : reinterpret_cast<const char *>(a.zero);
                lds_dma<16>(src, stage_lds + (unsigned)(buf * a.stage_chunks + c0) * 16u);
            }
            return;
        }
        for (int c0 = wave * 64; c0 < a.raw_chunks; c0 += NT) {
            const int c = c0 + lane;
            const int row = fast_div(c, a.magic_tw), tx = c - row * a.TW;
            const int half = fast_div(row, a.magic_rr), rr = row - half * a.RR;
            const int t = t0 + rr, db = fast_div(t, a.magic_thp);  // (t < THP + RR: small quotient)
            const int b = b0 + db, iy = t - db * a.THP - d.padU, ix = tx - d.padL;
            const int cb = cs * 2 + half;
            const bool ok = half < 2 && cb < a.in_cblocks && b < d.batch && iy >= 0 && iy < d.Hin && ix >= 0 && ix < d.Win;
            const char *src = ok ? reinterpret_cast<const char *>(Xb + (b * a.in_sb + cb * a.in_scb + iy * a.in_sy + ix * a.in_sx))
                                 : reinterpret_cast<const char *>(a.zero);
            lds_dma<16>(src, raw_lds + (unsigned)(buf * a.raw_chunks + c0) * 16u);
        }
    };
    // STAGED: staging slab -> raw slab.  One thread per chunk gathers the VEC channels of an input
    // position (consecutive lanes read consecutive columns) and writes them as 16 bytes; halo
    // columns become zeros.
    auto transpose = [&](int sbuf) {
        const T *sp = stage + (size_t)sbuf * a.stage_chunks * VEC;
        const int rw = a.RR * d.Win;
        for (int c = tid; c < 2 * a.PLANE; c += NT) {
            const int row = fast_div(c, a.magic_tw), tx = c - row * a.TW;
            const int half = fast_div(row, a.magic_rr), rr = row - half * a.RR;
            const int ix = tx - d.padL;
            union {
                uint4 v;
                T e[VEC];
            } u;
            u.v = make_uint4(0, 0, 0, 0);
            if (ix >= 0 && ix < d.Win) {
                const T *q = sp + (half * VEC) * rw + rr * d.Win + ix;
#pragma unroll
                for (int e = 0; e < VEC; ++e) u.e[e] = q[e * rw];
            }
            raw[c] = u.v;
        }
    };

    if ((int)blockIdx.x < a.tiles) enqueue(blockIdx.x, 0, 0);

    for (int i = tid; i < BN; i += NT) {
        int off = 0, h, w;
        if (m0 + i < a.g.M) axis_decode(a.g.c.m, m0 + i, off, h, w);
        mlut[i] = off;
    }
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

    // Accumulator element v of block j is filter j*32 + 8*(v/4) + 4*kg + v%4 (MFMA rows) at this
    // lane's pixel (MFMA column lr).
    T pend[FN][16];
    T *pend_out = nullptr;
    auto flush = [&]() {
        if (!pend_out) return;
        if (a.m_unit) {  // four consecutive filters of this pixel are four consecutive elements
#pragma unroll
            for (int j = 0; j < FN; ++j)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int ml = j * 32 + 8 * q + 4 * kg;
                    if (m0 + ml + 3 < a.g.M) {
                        typedef T t4 __attribute__((ext_vector_type(4)));
                        t4 o = {pend[j][4 * q], pend[j][4 * q + 1], pend[j][4 * q + 2], pend[j][4 * q + 3]};
                        *reinterpret_cast<t4 *>(pend_out + mlut[ml]) = o;
                    } else {
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            if (m0 + ml + e < a.g.M) pend_out[mlut[ml + e]] = pend[j][4 * q + e];
                    }
                }
            return;
        }
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int ml = j * 32 + 8 * (v >> 2) + 4 * kg + (v & 3);
                if (m0 + ml < a.g.M) pend_out[mlut[ml]] = pend[j][v];
            }
    };
    const int csteps = a.CinP / KSTEP;
    int buf = 0;
    for (int tile = blockIdx.x; tile < a.tiles; tile += gridDim.x) {
        // this lane's pixel: window corner in the raw tile, output offset
        const int n0 = tile * BM;
        const int b0 = n0 / PP, pix0 = n0 - b0 * PP, y0 = pix0 / d.Wo;
        const int p = min(n0 + wm * 32 + lr, a.g.N - 1);  // overhang pixels repeat the last one; never stored
        int pb, prem, py;
        if (a.fast_pix) {  // small quotients: pixel index relative to the tile's first sample
            const int q = pix0 + (p - n0), db = fast_div(q, a.magic_pp);
            pb = b0 + db;
            prem = q - db * PP;
            py = fast_div(prem, a.magic_wo);
        } else {
            pb = p / PP;
            prem = p - pb * PP;
            py = prem / d.Wo;
        }
        const int px = prem - py * d.Wo;
        const int corner = ((pb - b0) * a.THP + (py - y0) * d.sh) * a.TW + px * d.sw;
        int offn, h, w;
        if (a.nfast)
            offn = pb * a.g.c.n.o1 + prem * a.g.c.n.o0 + a.g.c.n.ob;
        else
            axis_decode(a.g.c.n, p, offn, h, w);

        f32x16 acc[FN];
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[j][v] = 0.f;

        for (int cs = 0; cs < csteps; ++cs, buf ^= 1) {
            wait_vmcnt<0>();
            __syncthreads();
            if (cs + 1 < csteps)
                enqueue(tile, cs + 1, buf ^ 1);
            else if (tile + (int)gridDim.x < a.tiles)
                enqueue(tile + gridDim.x, 0, buf ^ 1);
            if (cs == 0) flush();  // the previous tile's results
            if (STAGED) {
                transpose(buf);
                __syncthreads();
            }

            // Contraction, tap by tap.  Filters are the MFMA rows, pixels the columns: a lane ends
            // up with 16 filters of ONE pixel per block, so the 32 lanes of a half-wave store 32
            // consecutive pixels of a filter.
            const uint4 *prow = raw + (STAGED ? 0 : buf * a.raw_chunks) + corner + kg * a.PLANE;
            const char *frow = bl + lr * a.b_pitch + (cs * KSTEP + kg * VEC) * ES;
            for (int ky = 0; ky < d.KH; ++ky)
                for (int kx = 0; kx < d.KW; ++kx) {
                    const uint4 pf = prow[ky * a.TW + kx];
                    const char *fp = frow + (ky * d.KW + kx) * a.CinP * ES;
                    uint4 ff[FN];
#pragma unroll
                    for (int j = 0; j < FN; ++j) ff[j] = *reinterpret_cast<const uint4 *>(fp + j * 32 * a.b_pitch);
#pragma unroll
                    for (int j = 0; j < FN; ++j) mfma_step<T>(acc[j], ff[j], pf);
                }
        }

        // ---- results wait in registers until the next tile's loads are on their way (stores
        // count in vmcnt like loads: issued here, the wait at the top of the next iteration
        // would sit out their whole latency)
        pend_out = (n0 + wm * 32 + lr < a.g.N) ? reinterpret_cast<T *>(a.g.C) + offn : nullptr;
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) pend[j][v] = (T)acc[j][v];
    }
    flush();
}

// Channel-major [sample][channel][pixel] -> [sample][channel block][pixel] chunks of VEC channels
// (channels beyond the tensor are zeros).  One thread per chunk: its VEC element loads are
// coalesced along the pixels, its store is 16 bytes.
template <typename T>
__global__ __launch_bounds__(256) void chw_to_blocked_kernel(const T *__restrict__ in, uint4 *__restrict__ out, int C,
                                                             int cblocks, int HW, long long in_sb, long long in_sc,
                                                             long long total) {
    constexpr int VEC = 16 / (int)sizeof(T);
    // (the host keeps the chunk count below 2^31: 32-bit index arithmetic)
    const unsigned i = blockIdx.x * 256u + threadIdx.x;
    if (i >= total) return;
    const unsigned bc = i / (unsigned)HW;
    const int pix = (int)(i - bc * HW);
    const int b = (int)(bc / (unsigned)cblocks), cb = (int)(bc - (unsigned)b * cblocks);
    const T *src = in + b * in_sb + (long long)(cb * VEC) * in_sc + pix;
    union {
        uint4 v;
        T e[VEC];
    } u;
#pragma unroll
    for (int e = 0; e < VEC; ++e) u.e[e] = (cb * VEC + e < C) ? src[e * in_sc] : (T)0;
    out[i] = u.v;
}

template <typename T, int BM, int BN, bool STAGED>
static int launch_conv_tile(ConvTileArgs &a, size_t lds, hipStream_t s) {
    constexpr int NT = (BM / 32) * 64;
    auto kern = conv_tile_kernel<T, BM, BN, STAGED>;
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
    int occ = (int)((160 * 1024) / (lds + 2048));
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
    a.Wt = Wt;
    a.d = d;
    a.zero = st.zeros;
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
    if (!a.zero || d.padU < 0 || d.padD < 0 || d.padL < 0 || d.padR < 0) return -1;
    if (d.in_hwc ? (d.Cin % VEC != 0 || reinterpret_cast<uintptr_t>(X) % 16 != 0) : d.x_sy != d.Win) return -1;
    // every output pixel's window must lie inside the padded image
    if ((d.Ho - 1) * d.sh + d.KH > a.THP || (d.Wo - 1) * d.sw + d.KW > a.TW) return -1;
    const int cblocks = a.CinP / VEC;
    const long long in_chunks = (long long)d.batch * cblocks * d.Hin * d.Win;
    if (in_chunks >= ((long long)1 << 31)) return -1;

    // Raw rows of a tile: the output rows it spans (image seams included) plus the filter height.
    const int PP = d.Ho * d.Wo;
    a.RR = conv_raw_rows(BM, d.Ho, d.Wo, d.sh, d.KH, a.THP, a.g.N);
    if (a.RR > 64) return -1;
    a.PLANE = a.RR * a.TW;
    a.raw_chunks = (2 * a.PLANE + 63) & ~63;  // one slab: two channel blocks
    if (a.raw_chunks >= 65536 || a.TW >= 65536) return -1;
    int pitch16 = (d.KH * d.KW * a.CinP * ES + 15) / 16;
    if ((pitch16 & 1) == 0) ++pitch16;
    a.b_pitch = pitch16 * 16;

    // Staged route: the kernel copies pixel-major rows straight from the tensor and re-lays them in
    // LDS; it needs rows that are whole, aligned 16-byte groups.  Otherwise a first kernel writes
    // a blocked copy of the whole input.
    a.xg = d.Win / VEC;
    a.stage_chunks = (KSTEP * a.RR * a.xg + 63) & ~63;
    // It pays while slabs are small (one more barrier and an LDS-to-LDS pass per slab, and three
    // slab buffers instead of two: measured 12 against 15 us on 32x32 images with 16 channels,
    // 189 against 104 us on 56x56 with 32), so it is taken when a workgroup's slabs stay
    // below 40 KB.
    const bool staged = !d.in_hwc && d.Win % VEC == 0 && d.x_sc % VEC == 0 && d.x_sb % VEC == 0 &&
                        reinterpret_cast<uintptr_t>(X) % 16 == 0 && a.stage_chunks < 65536 &&
                        (long long)d.batch * d.x_sb < ((long long)1 << 31) &&
                        ((size_t)a.raw_chunks + 2 * (size_t)a.stage_chunks) * 16 <= 40 * 1024;
    a.magic_xg = magic_of(a.xg);
    a.magic_rrxg = magic_of(a.RR * a.xg);

    // Filters per workgroup: the narrowest of 32/64/128 that covers them (or 128 with several
    // column tiles), halved while the filter tile does not fit LDS (more column tiles, each
    // re-reading the pixels).  The kernel pays a per-workgroup price for its filter tile, so it
    // is only used when there are pixel tiles enough to give every CU a few workgroups.
    int bn = d.Cout <= 32 ? 32 : d.Cout <= 64 ? 64 : 128;
    size_t lds = 0;
    for (;; bn /= 2) {
        // filters + (one raw slab and two staging slabs | two raw slabs)
        lds = (size_t)bn * a.b_pitch +
              (staged ? (size_t)a.raw_chunks * 16 + 2 * (size_t)a.stage_chunks * 16 : 2 * (size_t)a.raw_chunks * 16);
        if (lds <= 150 * 1024 && (long)bn * d.KH * d.KW * cblocks < 65536) break;
        if (bn == 32) return -1;
    }
    a.b_bytes = bn * a.b_pitch;
    const long mt = (d.Cout + bn - 1) / bn;
    // ... or when the filter tile is small enough (20 KB) for that price not to matter: measured
    // 6.7 against 8.2 us for one 16->32 channel 32x32 sample, 19 against 8 us for eight 64->64 8x8 ones.
    if (st.gemm_path != 2 && ((long)(a.g.N + BM - 1) / BM) * mt < 2L * st.num_cu && a.b_bytes > 20 * 1024) return -1;

    a.magic_tw = magic_of(a.TW);
    a.magic_rr = magic_of(a.RR);
    a.magic_perm = magic_of(d.KH * d.KW * cblocks);
    a.magic_cb = magic_of(cblocks);
    a.magic_kw = magic_of(d.KW);
    a.fast_pix = (PP + BM < 65536 && d.Wo < 65536) ? 1 : 0;
    a.magic_pp = magic_of(PP);
    a.magic_wo = magic_of(d.Wo);
    a.magic_thp = magic_of(a.THP);
    if (a.THP + a.RR >= 65536) return -1;
    a.nfast = (c.n.d0 == PP && c.n.d1 >= (1 << 30)) ? 1 : 0;

    // 4-element stores along the filters: unit stride there, and every pixel's run 4-element aligned
    a.m_unit = (c.m.d0 >= c.m.n && c.m.o0 == 1 && (c.m.ob & 3) == 0 && c.n.d0 >= c.n.n && (c.n.o0 & 3) == 0 &&
                (c.n.ob & 3) == 0 && reinterpret_cast<uintptr_t>(Y) % (4 * sizeof(T)) == 0)
                   ? 1
                   : 0;
    if (d.in_hwc) {  // the tensor itself is the chunked input
        a.X = X;
        a.in_cblocks = d.Cin / VEC;
        a.in_sx = a.in_cblocks;
        a.in_sy = d.Win * a.in_cblocks;
        a.in_sb = d.Hin * a.in_sy;
        a.in_scb = 1;
        if ((long long)d.batch * a.in_sb >= ((long long)1 << 31)) return -1;
        if (bn == 128) return launch_conv_tile<T, BM, 128, false>(a, lds, st.stream);
        if (bn == 64) return launch_conv_tile<T, BM, 64, false>(a, lds, st.stream);
        return launch_conv_tile<T, BM, 32, false>(a, lds, st.stream);
    }
    a.in_cblocks = cblocks;
    a.in_sx = 1;
    a.in_sy = d.Win;
    a.in_scb = d.Hin * d.Win;
    a.in_sb = cblocks * a.in_scb;
    if (staged) {
        a.X = X;
        if (bn == 128) return launch_conv_tile<T, BM, 128, true>(a, lds, st.stream);
        if (bn == 64) return launch_conv_tile<T, BM, 64, true>(a, lds, st.stream);
        return launch_conv_tile<T, BM, 32, true>(a, lds, st.stream);
    }
    // re-lay the input in chunks of VEC channels
    uint4 *xb = reinterpret_cast<uint4 *>(workspace((size_t)in_chunks * 16));
    if (!xb) return 2;
    hipLaunchKernelGGL((chw_to_blocked_kernel<T>), dim3((unsigned)((in_chunks + 255) / 256)), dim3(256), 0, st.stream,
                       reinterpret_cast<const T *>(X), xb, d.Cin, cblocks, d.Hin * d.Win, d.x_sb, d.x_sc, in_chunks);
    if (!hip_ok(hipGetLastError(), "blocked layout launch")) return 2;
    a.X = xb;
    if (bn == 128) return launch_conv_tile<T, BM, 128, false>(a, lds, st.stream);
    if (bn == 64) return launch_conv_tile<T, BM, 64, false>(a, lds, st.stream);
    return launch_conv_tile<T, BM, 32, false>(a, lds, st.stream);
}

template int conv_tile<float>(const ConvTileDesc &, const void *, const void *, void *, const OutMap &);
template int conv_tile<half_t>(const ConvTileDesc &, const void *, const void *, void *, const OutMap &);

}  // namespace ptl
