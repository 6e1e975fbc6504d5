// Direct weight gradient of a channel-major convolution on MFMA.
//
// dW[co][ci][tap] = sum over pixels of dY[co][pixel] * X[ci][pixel shifted by tap]: a GEMM whose
// contraction runs over pixels.  A workgroup owns up to 64 output channels and a slab of CT
// input channels, walks pixel tiles (persistent, accumulators stay in registers) - a tile is
// R whole output rows of one sample, R the most that stays within 128 pixels, so that the
// input rows it needs are R + KH - 1 rows of the same sample - and per tile
//   * copies the dY rows of its output channels into LDS ([co][pixel], 16-byte loads);
//   * copies the input rows the tile touches into LDS as [ci][row][col] with a zero halo.
//     A thread loads 16 bytes of a row plus the two elements on either side and writes the
//     chunk once per filter column kx, shifted by kx elements, into a copy of the tile of its
//     own: every 16-byte store and every fragment load below is then 16-byte aligned (a
//     misaligned ds_read_b128 runs at a fraction of the aligned rate; measured 2.4x on the MFMA
//     loop).  When the copies do not fit there is one copy, stored behind the left halo with
//     unaligned 16-byte stores, and the fragment loads are unaligned.  Both copies are register-staged prefetches: the loads of tile t+1 are issued
//     before tile t is computed and parked in the other of two LDS buffers afterwards, one
//     barrier per tile;
//   * feeds the MFMAs: the dY fragment of a lane is one ds_read_b128 (8 pixels of one output
//     channel), the input fragment one ds_read_b128 at coloff(ci, tap) + pixoff(pixel group)
//     -- 8 consecutive pixels of a row shifted by the tap.  This needs unit column stride and
//     rows whose length is a multiple of the vector.
// The eight waves split the column blocks (ci, tap) four ways and the pixel groups two ways.
// Each workgroup leaves one fp32 partial of its dW block; a second kernel adds the partials.
#include "ptl_gemm_async.hpp"
#include "ptl_gemm_async.inc"
#include "ptl_conv_tile.hpp"
#include "ptl_host.hpp"

namespace ptl {

typedef unsigned int u4raw __attribute__((ext_vector_type(4)));
typedef u4raw u4_unaligned __attribute__((aligned(2)));

struct ConvWgArgs {
    const void *X;
    const void *dY;
    float *ws;  // [parts][Cout][Cin * taps]
    ConvTileDesc d;
    int CT;       // input channels per workgroup
    int TW, RR, PLANE;  // row pitch, rows and channel pitch of the input tile (elements; pitches multiples of the vector)
    int TWraw;    // input row with its halo (elements)
    int copies;   // copies of the input tile: KW (copy kx is shifted by kx elements) or 1
    int COPY;     // elements per copy
    int wchunks;  // whole 16-byte chunks of an input row
    int Wp;       // pixels a tile holds per output row: Wo rounded up to the vector
    int ragged;   // rows are not whole 16-byte chunks (4-byte aligned loads, short last chunk)
    int R;        // output rows per tile
    int tpi;      // tiles per sample
    int tiles;    // tiles of all samples
    int ksteps;   // MFMA steps that cover the R * Wo pixels of a tile
    int pitch_a;  // bytes per dY row in LDS
    int a_bytes;  // LDS bytes of the dY tile (the input tile follows)
    int raw_bytes;
    int cblocks;  // 32-wide column blocks of (ci, tap) per workgroup
    int xg;       // 16-byte chunks per row of the input tile
    unsigned magic_xg, magic_rr, magic_taps, magic_kw, magic_tpi, magic_wp;
};

// Two elements as a pair of dwords (fp16: one dword, the second unused).
template <typename T>
__device__ inline uint2 load_two(const T *p) {
    if constexpr (sizeof(T) == 2) return make_uint2(*reinterpret_cast<const unsigned *>(p), 0u);
    else return *reinterpret_cast<const uint2 *>(p);
}

// The first `n` (2, 4, 6 or 8) fp16 elements at a 4-byte aligned address, the rest zero.
__device__ inline uint4 load_upto8(const half_t *p, int n) {
    if (n == 8) {
        const u4raw w = *reinterpret_cast<const u4raw __attribute__((aligned(4))) *>(p);
        return make_uint4(w.x, w.y, w.z, w.w);
    }
    const unsigned *q = reinterpret_cast<const unsigned *>(p);
    uint4 v = make_uint4(0, 0, 0, 0);
    if (n >= 2) v.x = q[0];
    if (n >= 4) v.y = q[1];
    if (n >= 6) v.z = q[2];
    return v;
}

// The 16 bytes that start `shift` elements (-2..2) after the chunk `cur`, given the two elements before
// and after it.
template <typename T>
__device__ inline uint4 shifted_chunk(const uint2 &before, const uint4 &cur, const uint2 &after, int shift) {
    if constexpr (sizeof(T) == 2) {
        const unsigned w0 = before.x, w1 = cur.x, w2 = cur.y, w3 = cur.z, w4 = cur.w, w5 = after.x;
        switch (shift) {
            case -2: return make_uint4(w0, w1, w2, w3);
            case -1:
                return make_uint4(__builtin_amdgcn_alignbit(w1, w0, 16), __builtin_amdgcn_alignbit(w2, w1, 16),
                                  __builtin_amdgcn_alignbit(w3, w2, 16), __builtin_amdgcn_alignbit(w4, w3, 16));
            case 1:
                return make_uint4(__builtin_amdgcn_alignbit(w2, w1, 16), __builtin_amdgcn_alignbit(w3, w2, 16),
                                  __builtin_amdgcn_alignbit(w4, w3, 16), __builtin_amdgcn_alignbit(w5, w4, 16));
            case 2: return make_uint4(w2, w3, w4, w5);
            default: return cur;
        }
    } else {
        switch (shift) {
            case -2: return make_uint4(before.x, before.y, cur.x, cur.y);
            case -1: return make_uint4(before.y, cur.x, cur.y, cur.z);
            case 1: return make_uint4(cur.y, cur.z, cur.w, after.x);
            case 2: return make_uint4(cur.z, cur.w, after.x, after.y);
            default: return cur;
        }
    }
}

// SHIFTED: one copy of the input tile per filter column (a.copies > 1); 2: three filter columns with one column of
// left padding, the shifts -1, 0, 1 known to the compiler; 3: the same for rows that are not whole 16-byte chunks
// (fp16, even row lengths: a tile holds every output row padded to whole chunks, the pad pixels with zero dY).
template <typename T, int RB, int CBW, int SHIFTED>
__global__ __launch_bounds__(512) void conv_wg_kernel(const ConvWgArgs a) {
    constexpr int NT = 512, KT = 128, MAX_COPIES = 5;
    constexpr int ES = (int)sizeof(T), VEC = 16 / ES, KSTEP = 2 * VEC, GROUPS = KT / VEC;
    constexpr bool RAGGED = SHIFTED == 3, FIXED3 = SHIFTED >= 2;
    extern __shared__ __attribute__((aligned(16))) char smem[];
    // two buffers, each: dY tile [32*RB][pitch_a] followed by the copies of the input tile [copy][CT][RR][TW]
    const int buf_bytes = a.a_bytes + a.raw_bytes;
    __shared__ int pixoff[GROUPS];  // per pixel group: offset of its first pixel in the input tile (the same in every tile)

    const ConvTileDesc &d = a.d;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wk = wave & 1, wc = wave >> 1;
    const int kg = lane >> 5, lr = lane & 31;
    const int c0 = blockIdx.y * a.CT, r0 = blockIdx.z * 32 * RB;
    const int PP = d.Ho * d.Wo, taps = d.KH * d.KW;
    const int cols = a.CT * taps;  // column m' = ci_local * taps + tap
    const T *__restrict__ X = reinterpret_cast<const T *>(a.X);
    const T *__restrict__ dY = reinterpret_cast<const T *>(a.dY);

    // this lane's column in each of its blocks: offset of (ci, tap) inside the input tile
    int coloff[CBW];
#pragma unroll
    for (int jj = 0; jj < CBW; ++jj) {
        int m = (wc + 4 * jj) * 32 + lr;
        if (m >= cols) m = cols - 1;  // surplus columns repeat the last one; never stored
        const int ci = fast_div(m, a.magic_taps), tap = m - ci * taps;
        const int ky = fast_div(tap, a.magic_kw), kx = tap - ky * d.KW;
        coloff[jj] = ci * a.PLANE + ky * a.TW + (SHIFTED ? kx * a.COPY : kx);
    }

    f32x16 acc[RB][CBW];
#pragma unroll
    for (int r = 0; r < RB; ++r)
#pragma unroll
        for (int jj = 0; jj < CBW; ++jj)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[r][jj][v] = 0.f;

    // Both input tiles start as zeros: the padding between rows and channels is never written again,
    // everything else is rewritten for every tile (rows outside the image, columns of the halo and
    // channels beyond the tensor as zeros).
    for (int b = 0; b < 2; ++b)
        for (int c = tid; c < a.raw_bytes / 16; c += NT)
            reinterpret_cast<uint4 *>(smem + b * buf_bytes + a.a_bytes)[c] = make_uint4(0, 0, 0, 0);
    if (tid < GROUPS) {
        // groups past the tile's pixels (their dY is zero) read the start of the tile
        const int p = tid * VEC < a.R * a.Wp ? tid * VEC : 0;
        const int y = fast_div(p, a.magic_wp);
        pixoff[tid] = y * d.sh * a.TW + (p - y * a.Wp);
    }
    __syncthreads();

    // Register-staged prefetch: the global loads of tile t+1 are issued before tile t is
    // computed and stored to the other LDS buffer afterwards; one barrier per tile.
    // What a thread copies is the same piece of every tile - the chunk (row, pixel group) of
    // the dY tile, the unit (ci, tile row, chunk) of the input tile - so its decoding is
    // done once here; per tile only the sample and the first row change.
    constexpr int A_CHUNKS = 32 * RB * (KT / VEC);
    constexpr int A_PER = (A_CHUNKS + NT - 1) / NT;  // dY chunks per thread
    const int units = a.CT * a.RR * a.xg;            // (ci, tile row, chunk of VEC columns)
    constexpr int U_MAX = 4;                         // input units per thread the registers hold (host checks)
    uint4 regA[A_PER], regU[U_MAX];
    uint2 regP[SHIFTED ? U_MAX : 1], regN[SHIFTED ? U_MAX : 1];  // the two elements before and after the chunk
    // Offsets are 32-bit (the host checks that one sample fits) on top of a base that is the same for
    // the whole workgroup, so that the loads take the scalar-base form without 64-bit address sums.
    int a_lds[A_PER], a_y[A_PER];    // LDS byte offset (-1: no chunk), output row inside the tile
    int a_n[RAGGED ? A_PER : 1];     // elements of the chunk that lie inside the row
    unsigned a_row[A_PER];           // element offset of (output channel, pixel group) inside the sample
    bool a_ok[A_PER];
    int u_lds[U_MAX], u_rr[U_MAX];   // LDS byte offset (-1: no unit), tile row
    int u_has[U_MAX];                // 1: the chunk lies inside the row, 2: the elements before it, 4: those after it;
                                     // 0: channel beyond the tensor
    unsigned u_src[U_MAX];           // element offset of (channel, tile row, chunk) from the tile's first row
    int u_n[RAGGED ? U_MAX : 1];     // elements of the chunk that lie inside the row
    const int uslots = (units + NT - 1) / NT;
#pragma unroll
    for (int i = 0; i < A_PER; ++i) {
        const int c = tid + i * NT;
        const int row = c / (KT / VEC), g = c % (KT / VEC);
        a_lds[i] = c < A_CHUNKS ? row * a.pitch_a + g * 16 : -1;
        a_y[i] = fast_div(g * VEC, a.magic_wp);
        const int x = g * VEC - a_y[i] * a.Wp;
        a_ok[i] = c < A_CHUNKS && r0 + row < d.Cout && x < d.Wo;
        a_row[i] = a_ok[i] ? (unsigned)((r0 + row) * PP + a_y[i] * d.Wo + x) : 0u;
        if constexpr (RAGGED) a_n[i] = d.Wo - x < VEC ? d.Wo - x : VEC;
    }
#pragma unroll
    for (int i = 0; i < U_MAX; ++i) {
        const int u = tid + i * NT;
        const int row = fast_div(u, a.magic_xg), xg = u - row * a.xg;
        const int ci = fast_div(row, a.magic_rr), rr = row - ci * a.RR;
        u_lds[i] = u < units ? (ci * a.PLANE + rr * a.TW + xg * VEC) * ES : -1;
        u_rr[i] = rr;
        u_has[i] = (xg * VEC < d.Win ? 1 : 0) | (xg >= 1 && xg * VEC - 2 < d.Win ? 2 : 0) | (xg * VEC + VEC < d.Win ? 4 : 0);
        if (!SHIFTED) {  // the chunks of the row go behind the left halo as they are
            u_has[i] &= 1;
            u_lds[i] = (u < units && xg < a.wchunks) ? u_lds[i] + d.padL * ES : -1;
        }
        if (u >= units || c0 + ci >= d.Cin) u_has[i] = 0;
        u_src[i] = u_has[i] ? (unsigned)((c0 + ci) * (int)d.x_sc + rr * (int)d.x_sy + xg * VEC) : 0u;
        if constexpr (RAGGED) u_n[i] = d.Win - xg * VEC < VEC ? d.Win - xg * VEC : VEC;
    }

    auto fetch = [&](int tile) {
        const int b0 = fast_div(tile, a.magic_tpi), y0 = (tile - b0 * a.tpi) * a.R;
        const int rows = d.Ho - y0 < a.R ? d.Ho - y0 : a.R;  // the last tile of a sample may be short
        const int raw_rows = (rows - 1) * d.sh + d.KH, t0 = y0 * d.sh - d.padU;
        // tile rows [lo, hi) lie inside the image and are needed by the tile's pixels
        const int lo = t0 < 0 ? -t0 : 0, hi = d.Hin - t0 < raw_rows ? d.Hin - t0 : raw_rows;
        const T *gy = dY + (long long)b0 * d.Cout * PP + (long long)y0 * d.Wo;
        const T *gx = X + (long long)b0 * d.x_sb + (long long)t0 * d.x_sy;  // dereferenced for rows of the image only
#pragma unroll
        for (int i = 0; i < A_PER; ++i) {
            regA[i] = make_uint4(0, 0, 0, 0);
            if (a_ok[i] && a_y[i] < rows) {
                if constexpr (RAGGED) regA[i] = load_upto8(gy + a_row[i], a_n[i]);
                else regA[i] = *reinterpret_cast<const uint4 *>(gy + a_row[i]);
            }
        }
#pragma unroll
        for (int i = 0; i < U_MAX; ++i) {
            if (i >= uslots) break;
            regU[i] = make_uint4(0, 0, 0, 0);
            if constexpr (SHIFTED) regP[i] = regN[i] = make_uint2(0, 0);
            if (u_has[i] && u_rr[i] >= lo && u_rr[i] < hi) {
                const T *src = gx + u_src[i];
                if (u_has[i] & 1) {
                    if constexpr (RAGGED) regU[i] = load_upto8(src, u_n[i]);
                    else regU[i] = *reinterpret_cast<const uint4 *>(src);
                }
                if constexpr (SHIFTED) {
                    if (u_has[i] & 2) regP[i] = load_two<T>(src - 2);
                    if (u_has[i] & 4) regN[i] = load_two<T>(src + VEC);
                }
            }
        }
    };
    auto park = [&](int buf) {
        char *at = smem + buf * buf_bytes;
        char *raw = at + a.a_bytes;
#pragma unroll
        for (int i = 0; i < A_PER; ++i)
            if (a_lds[i] >= 0) *reinterpret_cast<uint4 *>(at + a_lds[i]) = regA[i];
        if constexpr (!SHIFTED) {
#pragma unroll
            for (int i = 0; i < U_MAX; ++i) {
                if (i >= uslots) break;
                if (u_lds[i] >= 0) {
                    u4raw w = {regU[i].x, regU[i].y, regU[i].z, regU[i].w};
                    *reinterpret_cast<u4_unaligned *>(raw + u_lds[i]) = w;
                }
            }
        } else {
#pragma unroll
            for (int s = 0; s < (FIXED3 ? 3 : MAX_COPIES); ++s) {
                if (!FIXED3 && s >= a.copies) break;
                // copy s, position i holds input column i + s - padL
#pragma unroll
                for (int i = 0; i < U_MAX; ++i) {
                    if (i >= uslots) break;
                    if (u_lds[i] >= 0)
                        *reinterpret_cast<uint4 *>(raw + s * a.COPY * ES + u_lds[i]) =
                            shifted_chunk<T>(regP[i], regU[i], regN[i], FIXED3 ? s - 1 : s - d.padL);
                }
            }
        }
    };

    int buf = 0;
    if ((int)blockIdx.x < a.tiles) fetch(blockIdx.x);
    for (int tile = blockIdx.x; tile < a.tiles; tile += gridDim.x, buf ^= 1) {
        park(buf);
        __syncthreads();  // tile parked; every wave is done with the tile before the previous one (same buffer)
        if (tile + (int)gridDim.x < a.tiles) fetch(tile + gridDim.x);
        const char *at = smem + buf * buf_bytes;
        const T *raw = reinterpret_cast<const T *>(at + a.a_bytes);
        for (int ks = wk; ks < a.ksteps; ks += 2) {
            const int po = pixoff[ks * 2 + kg];
            uint4 af[RB];
#pragma unroll
            for (int r = 0; r < RB; ++r)
                af[r] = *reinterpret_cast<const uint4 *>(at + (r * 32 + lr) * a.pitch_a + (ks * KSTEP + kg * VEC) * ES);
#pragma unroll
            for (int jj = 0; jj < CBW; ++jj) {
                if (wc + 4 * jj >= a.cblocks) continue;
                const u4raw w = *reinterpret_cast<const u4_unaligned *>(raw + coloff[jj] + po);
                const uint4 bf = make_uint4(w.x, w.y, w.z, w.w);
#pragma unroll
                for (int r = 0; r < RB; ++r) mfma_step<T>(acc[r][jj], af[r], bf);
            }
        }
    }
    __syncthreads();

    // the two pixel-group halves meet in LDS (one block of 32 output channels at a time, so that the
    // exchange fits the space of the tiles), then one fp32 partial per workgroup
    float *red = reinterpret_cast<float *>(smem);
    constexpr int PER = CBW * 16;
    const int Kw = d.Cin * taps;
    const int valid_cols = (d.Cin - c0 < a.CT ? d.Cin - c0 : a.CT) * taps;
    float *__restrict__ out = a.ws + (size_t)blockIdx.x * d.Cout * Kw + (size_t)c0 * taps;
#pragma unroll
    for (int r = 0; r < RB; ++r) {
        float *mine = red + (size_t)wc * PER * 64 + lane;
        if (wk == 1) {
#pragma unroll
            for (int jj = 0; jj < CBW; ++jj)
#pragma unroll
                for (int v = 0; v < 16; ++v) mine[(jj * 16 + v) * 64] = acc[r][jj][v];
        }
        __syncthreads();
        if (wk == 0) {
#pragma unroll
            for (int jj = 0; jj < CBW; ++jj) {
                const int m = (wc + 4 * jj) * 32 + lr;
                if (wc + 4 * jj >= a.cblocks || m >= valid_cols) continue;
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const int co = r0 + r * 32 + 8 * (v >> 2) + 4 * kg + (v & 3);
                    if (co < d.Cout) out[(size_t)co * Kw + m] = acc[r][jj][v] + mine[(jj * 16 + v) * 64];
                }
            }
        }
        if (r + 1 < RB) __syncthreads();
    }
}

// dW[i] = sum over parts of ws[part][i]: 64 outputs per workgroup, 16 part groups in parallel,
// eight loads in flight per thread (the partials are a few MB spread over hundreds of parts:
// the kernel lives on memory-level parallelism, not on arithmetic).
template <typename T>
__global__ __launch_bounds__(1024) void conv_wg_reduce_kernel(const float *__restrict__ ws, T *__restrict__ dW, int total,
                                                              int parts) {
    __shared__ float part_sum[16][64];
    const int o = threadIdx.x & 63, pg = threadIdx.x >> 6;
    const int i = blockIdx.x * 64 + o;
    float s = 0.f;
    if (i < total) {
        const float *src = ws + i;
        int p = pg;
        for (; p + 7 * 16 < parts; p += 8 * 16) {
            float v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = src[(size_t)(p + u * 16) * total];
#pragma unroll
            for (int u = 0; u < 8; ++u) s += v[u];
        }
        for (; p < parts; p += 16) s += src[(size_t)p * total];
    }
    part_sum[pg][o] = s;
    __syncthreads();
    if (pg == 0 && i < total) {
#pragma unroll
        for (int q = 1; q < 16; ++q) s += part_sum[q][o];
        dW[i] = (T)s;
    }
}

// The same sum for few parts of a large tensor: four consecutive outputs per thread, 16-byte loads, all
// parts of a thread in flight together.
template <typename T>
__global__ __launch_bounds__(256) void conv_wg_reduce_few_kernel(const float *__restrict__ ws, T *__restrict__ dW,
                                                                 int total, int parts) {
    const int i = (blockIdx.x * 256 + threadIdx.x) * 4;
    if (i >= total) return;
    const float4 *src = reinterpret_cast<const float4 *>(ws + i);
    const size_t step = (size_t)total / 4;
    float4 s = make_float4(0.f, 0.f, 0.f, 0.f);
    int p = 0;
    for (; p + 8 <= parts; p += 8) {
        float4 v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = src[(size_t)(p + u) * step];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            s.x += v[u].x;
            s.y += v[u].y;
            s.z += v[u].z;
            s.w += v[u].w;
        }
    }
    for (; p < parts; ++p) {
        const float4 v = src[(size_t)p * step];
        s.x += v.x;
        s.y += v.y;
        s.z += v.z;
        s.w += v.w;
    }
    typedef T t4 __attribute__((ext_vector_type(4)));
    const t4 o = {(T)s.x, (T)s.y, (T)s.z, (T)s.w};
    *reinterpret_cast<t4 *>(dW + i) = o;
}

template <typename T, int RB, int CBW>
static int launch_conv_wg(ConvWgArgs &a, int gy, int gz, void *dW, hipStream_t s) {
    constexpr int ES = (int)sizeof(T), VEC = 16 / ES;
    a.pitch_a = 128 * ES + 16;
    a.a_bytes = 32 * RB * a.pitch_a;
    const size_t red = (size_t)4 * CBW * 16 * 64 * 4;  // exchange of one 32-channel block between the wave pairs
    // (fp16; an fp32 fragment feeds four MFMAs and the extra registers would cost a workgroup per CU)
    // one shifted copy of the input tile per filter column when the chunk shifts are within the two elements
    // a thread holds on either side and both buffers fit (pitches in whole chunks, one odd chunk per channel to
    // spread the channels over the LDS banks); else one copy with the pitches of the data and unaligned
    // fragment loads
    const int KW = a.d.KW, first = -a.d.padL, last = KW - 1 - a.d.padL;
    size_t lds = 0;
    for (a.copies = (ES == 2 && KW > 1 && KW <= 5 && first >= -2 && last <= 2) ? KW : 1;; a.copies = 1) {
        a.TW = a.copies > 1 ? (a.TWraw + VEC - 1) / VEC * VEC : a.TWraw;
        a.PLANE = a.RR * a.TW + (a.copies > 1 ? VEC : 0);
        a.COPY = a.CT * a.PLANE;
        a.xg = a.copies > 1 ? a.TW / VEC : a.wchunks;
        if (a.ragged && a.copies == 1) return -1;  // short chunks exist in the shifted form only
        // slack: an unaligned fragment may start at the last element
        a.raw_bytes = (int)((((size_t)a.copies * a.COPY * ES + 32) + 15) & ~(size_t)15);
        lds = 2 * ((size_t)a.a_bytes + a.raw_bytes);
        if (lds <= 150 * 1024 || a.copies == 1) break;
    }
    a.magic_xg = magic_of(a.xg);
    if ((long)a.CT * a.RR * a.xg > 4L * 512) return -1;  // input units per thread that the prefetch registers hold
    if (lds < red) lds = red;
    if (lds > 150 * 1024) return -1;
    constexpr bool CAN_SHIFT = ES == 2;
    const int mode = !(CAN_SHIFT && a.copies > 1) ? 0 : (KW == 3 && a.d.padL == 1) ? (a.ragged ? 3 : 2) : 1;
    if (a.ragged && mode != 3) return -1;
    auto kern = mode == 3   ? conv_wg_kernel<T, RB, CBW, CAN_SHIFT ? 3 : 0>
                : mode == 2 ? conv_wg_kernel<T, RB, CBW, CAN_SHIFT ? 2 : 0>
                : mode == 1 ? conv_wg_kernel<T, RB, CBW, CAN_SHIFT ? 1 : 0>
                            : conv_wg_kernel<T, RB, CBW, 0>;
    static bool attr_set[4] = {false, false, false, false};
    if (!attr_set[mode]) {
        if (!hip_ok(hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, 150 * 1024),
                    "hipFuncSetAttribute"))
            return 2;
        attr_set[mode] = true;
    }
    // as many workgroups as the CUs hold at once over the whole grid, each walking an equal share of the pixel tiles
    long parts = (lds <= 80 * 1024 ? 2L : 1L) * state().num_cu / ((long)gy * gz);
    // (fp16 with under four tiles per workgroup: half as many partial sums to write and add pay more than the
    // second workgroup per CU; measured 14.5 against 16.7 us for 16 -> 32 channels, 32x32, batch 128)
    if (ES == 2 && parts > 1 && a.tiles < 4 * parts) parts = (parts + 1) / 2;
    if (parts < 1) parts = 1;
    if (parts > a.tiles) parts = a.tiles;
    const int per = (int)((a.tiles + parts - 1) / parts);
    parts = (a.tiles + per - 1) / per;
    const int total = a.d.Cout * a.d.Cin * a.d.KH * a.d.KW;
    a.ws = workspace((size_t)parts * total * sizeof(float));
    if (!a.ws) return 2;
    // a workgroup writes only the columns of its own channel slab; with one slab per row the
    // partial is complete, otherwise every (slab, row tile) pair writes a disjoint part of it
    hipLaunchKernelGGL(kern, dim3((unsigned)parts, gy, gz), dim3(512), lds, s, a);
    if (!hip_ok(hipGetLastError(), "conv wg launch")) return 2;
    if (parts <= 32 && total % 4 == 0 && total >= 65536 && reinterpret_cast<uintptr_t>(dW) % (4 * sizeof(T)) == 0)
        hipLaunchKernelGGL((conv_wg_reduce_few_kernel<T>), dim3((total / 4 + 255) / 256), dim3(256), 0, s, a.ws,
                           reinterpret_cast<T *>(dW), total, (int)parts);
    else
        hipLaunchKernelGGL((conv_wg_reduce_kernel<T>), dim3((total + 63) / 64), dim3(1024), 0, s, a.ws,
                           reinterpret_cast<T *>(dW), total, (int)parts);
    return hip_ok(hipGetLastError(), "conv wg reduce launch") ? 0 : 2;
}

template <typename T>
int conv_tile_wg(const ConvTileDesc &d, const void *X, const void *dY, void *dW) {
    State &st = state();
    constexpr int ES = (int)sizeof(T), VEC = 16 / ES;
    ConvWgArgs a = {};
    a.X = X;
    a.dY = dY;
    a.d = d;
    const int THP = d.Hin + d.padU + d.padD, TWraw = d.Win + d.padL + d.padR;
    if (d.padU < 0 || d.padD < 0 || d.padL < 0 || d.padR < 0) return -1;
    if ((d.Ho - 1) * d.sh + d.KH > THP || (d.Wo - 1) * d.sw + d.KW > TWraw) return -1;
    // 8 (4) consecutive pixels of a fragment must be 8 consecutive input columns of one row,
    // and input rows must be copyable 16 bytes at a time
    if (d.sw != 1) return -1;
    a.ragged = d.Wo % VEC || d.Win % VEC || d.x_sy % VEC || d.x_sc % VEC || d.x_sb % VEC ||
               reinterpret_cast<uintptr_t>(X) % 16 || reinterpret_cast<uintptr_t>(dY) % 16;
    // ... or, for fp16 3x3 layers with one column of padding, rows of whole dwords
    if (a.ragged && (ES != 2 || d.KW != 3 || d.padL != 1 || d.Wo % 2 || d.Win % 2 || d.x_sy % 2 || d.x_sc % 2 ||
                     d.x_sb % 2 || reinterpret_cast<uintptr_t>(X) % 4 || reinterpret_cast<uintptr_t>(dY) % 4))
        return -1;
    a.Wp = (d.Wo + VEC - 1) / VEC * VEC;
    if (a.Wp > 128) return -1;  // a tile is whole output rows within 128 pixels
    // offsets inside one sample are 32-bit
    if ((long long)d.Cin * d.x_sc + (long long)(d.Hin + d.KH) * d.x_sy >= ((long long)1 << 31) ||
        (long long)d.Cout * d.Ho * d.Wo >= ((long long)1 << 31) || d.x_sc >= ((long long)1 << 31))
        return -1;
    a.R = 128 / a.Wp < d.Ho ? 128 / a.Wp : d.Ho;
    a.tpi = (d.Ho + a.R - 1) / a.R;
    if ((long long)d.batch * a.tpi * a.tpi >= ((long long)1 << 32)) return -1;  // range of the reciprocal division
    a.tiles = d.batch * a.tpi;
    a.ksteps = (a.R * a.Wp + 2 * VEC - 1) / (2 * VEC);
    // few pixel tiles: worth it only for small fp16 weight tensors (measured 8.6 against 11.2 us for one
    // 16->32 channel 32x32 sample, 14 against 9.5 us for eight 64->64 8x8 ones)
    // (from 128 channels on the alternative is the sum over taps, which loses from half a tile per CU:
    // measured 25 against 33 us for 128 -> 128 channels on 8x8 images at batch 128)
    // (with 256 channels on both sides a tile carries enough work at any count: 12 against 29 us for eight
    // 256 -> 256 7x7 samples; otherwise from half a tile per CU: 32 against 43 us through the gathering GEMM for
    // 128 -> 64 channels on 28x28 at batch 32, 21 against 14 us at batch 8)
    const bool wide = d.Cin >= 128 && d.Cout >= 128 && 2 * a.tiles >= st.num_cu;
    const bool deep = d.Cin >= 256 && d.Cout >= 256;
    if (st.gemm_path != 2 && 2 * a.tiles < st.num_cu && !wide && !deep &&
        !(ES == 2 && (long)d.Cout * d.Cin * d.KH * d.KW <= 8192))
        return -1;

    const int taps = d.KH * d.KW;
    a.TWraw = TWraw;
    a.RR = (a.R - 1) * d.sh + d.KH;
    if (a.RR > 64) return -1;
    a.CT = d.Cin <= 16 ? 16 : 32;
    a.wchunks = d.Win / VEC;
    if ((long)a.CT * a.RR * (TWraw / VEC + 1) >= 65536 || (long)a.CT * taps >= 65536) return -1;
    a.cblocks = (a.CT * taps + 31) / 32;
    a.magic_rr = magic_of(a.RR);
    a.magic_taps = magic_of(taps);
    a.magic_kw = magic_of(d.KW);
    a.magic_tpi = magic_of(a.tpi);
    a.magic_wp = magic_of(a.Wp);
    const int gy = (d.Cin + a.CT - 1) / a.CT;
    const int cbw = (a.cblocks + 3) / 4;  // column blocks per wave
    if (cbw > 3) return -1;
    if (d.Cout <= 32) {
        const int gz = 1;
        if (cbw == 1) return launch_conv_wg<T, 1, 1>(a, gy, gz, dW, st.stream);
        if (cbw == 2) return launch_conv_wg<T, 1, 2>(a, gy, gz, dW, st.stream);
        return launch_conv_wg<T, 1, 3>(a, gy, gz, dW, st.stream);
    }
    const int gz = (d.Cout + 63) / 64;
    if (cbw == 1) return launch_conv_wg<T, 2, 1>(a, gy, gz, dW, st.stream);
    if (cbw == 2) return launch_conv_wg<T, 2, 2>(a, gy, gz, dW, st.stream);
    return launch_conv_wg<T, 2, 3>(a, gy, gz, dW, st.stream);
}

template int conv_tile_wg<float>(const ConvTileDesc &, const void *, const void *, void *);
template int conv_tile_wg<half_t>(const ConvTileDesc &, const void *, const void *, void *);

}  // namespace ptl
