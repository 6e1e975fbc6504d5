// Direct weight gradient of a channel-major convolution on MFMA.
//
// dW[co][ci][tap] = sum over pixels of dY[co][pixel] * X[ci][pixel shifted by tap]: a GEMM whose
// contraction runs over pixels.  A workgroup owns up to 64 output channels and a slab of CT
// input channels, walks pixel tiles of 128 (persistent, accumulators stay in registers) and
// per tile
//   * copies the dY rows of its output channels into LDS ([co][pixel], 16-byte loads);
//   * copies the input rows the tile touches into LDS as [ci][row][col] with a zero halo,
//     16 bytes at a time (the halo makes the destination 2-byte aligned only; LDS takes
//     unaligned 16-byte stores and loads).  Both copies are register-staged prefetches: the
//     loads of tile t+1 are issued before tile t is computed and parked in the other of two
//     LDS buffers afterwards, one barrier per tile;
//   * feeds the MFMAs: the dY fragment of a lane is one aligned ds_read_b128 (8 pixels of one
//     output channel), the input fragment one unaligned ds_read_b128 at
//     coloff(ci, tap) + pixoff(pixel group) -- 8 consecutive pixels of a row shifted by the
//     tap.  This needs unit column stride and rows whose length is a multiple of the vector.
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
    int THP, TW, RR, PLANE;
    int tiles;    // pixel tiles of 128
    int N;        // pixels
    int pitch_a;  // bytes per dY row in LDS
    int a_bytes;  // LDS bytes of the dY tile (the raw tile follows)
    int raw_bytes;
    int cblocks;  // 32-wide column blocks of (ci, tap) per workgroup
    int xg;       // 16-byte groups per input row
    unsigned magic_xg, magic_rr, magic_taps, magic_kw, magic_thp;
};

template <typename T, int RB, int CBW>
__global__ __launch_bounds__(512) void conv_wg_kernel(const ConvWgArgs a) {
    constexpr int NT = 512, KT = 128;
    constexpr int ES = (int)sizeof(T), VEC = 16 / ES, KSTEP = 2 * VEC, KSTEPS = KT / KSTEP, GROUPS = KT / VEC;
    extern __shared__ __attribute__((aligned(16))) char smem[];
    // two buffers, each: dY tile [32*RB][pitch_a] followed by the input tile [CT][RR][TW]
    const int buf_bytes = a.a_bytes + a.raw_bytes;
    __shared__ int pixoff[2][GROUPS];  // per pixel group: raw offset of its first pixel

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

    // this lane's column in each of its blocks: offset of (ci, tap) inside the raw tile
    int coloff[CBW];
#pragma unroll
    for (int jj = 0; jj < CBW; ++jj) {
        int m = (wc + 4 * jj) * 32 + lr;
        if (m >= cols) m = cols - 1;  // surplus columns repeat the last one; never stored
        const int ci = fast_div(m, a.magic_taps), tap = m - ci * taps;
        const int ky = fast_div(tap, a.magic_kw), kx = tap - ky * d.KW;
        coloff[jj] = ci * a.PLANE + ky * a.TW + kx;
    }

    f32x16 acc[RB][CBW];
#pragma unroll
    for (int r = 0; r < RB; ++r)
#pragma unroll
        for (int jj = 0; jj < CBW; ++jj)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[r][jj][v] = 0.f;

    // Both input tiles start as zeros: the halo columns are never written again, everything
    // else is rewritten for every tile (rows outside the image and channels beyond the tensor
    // as zeros).
    for (int b = 0; b < 2; ++b)
        for (int c = tid; c < a.raw_bytes / 16; c += NT)
            reinterpret_cast<uint4 *>(smem + b * buf_bytes + a.a_bytes)[c] = make_uint4(0, 0, 0, 0);
    __syncthreads();

    // Register-staged prefetch: the global loads of tile t+1 are issued before tile t is
    // computed and stored to the other LDS buffer afterwards; one barrier per tile.
    constexpr int A_CHUNKS = 32 * RB * (KT / VEC);
    constexpr int A_PER = (A_CHUNKS + NT - 1) / NT;  // dY chunks per thread
    const int units = a.CT * a.RR * a.xg;            // (ci, raw row, group of VEC columns)
    constexpr int U_MAX = 4;                         // input units per thread the registers hold (host checks)
    uint4 regA[A_PER], regU[U_MAX];

    auto fetch = [&](int tile) {
        const int n0 = tile * KT;
        const int b0 = n0 / PP, pix0 = n0 - b0 * PP, y0 = pix0 / d.Wo;
        const int t0 = y0 * d.sh;
#pragma unroll
        for (int i = 0; i < A_PER; ++i) {
            const int c = tid + i * NT;
            const int row = c / (KT / VEC), g = c % (KT / VEC);
            int q = pix0 + g * VEC, b = b0;
            while (q >= PP) {
                q -= PP;
                ++b;
            }
            regA[i] = make_uint4(0, 0, 0, 0);
            if (c < A_CHUNKS && n0 + g * VEC < a.N && r0 + row < d.Cout)
                regA[i] = *reinterpret_cast<const uint4 *>(dY + ((long long)b * d.Cout + r0 + row) * PP + q);
        }
#pragma unroll
        for (int i = 0; i < U_MAX; ++i) {
            const int u = tid + i * NT;
            regU[i] = make_uint4(0, 0, 0, 0);
            if (u < units) {
                const int row = fast_div(u, a.magic_xg), xg = u - row * a.xg;
                const int ci = fast_div(row, a.magic_rr), rr = row - ci * a.RR;
                const int t = t0 + rr, db = fast_div(t, a.magic_thp);
                const int b = b0 + db, iy = t - db * a.THP - d.padU;
                if (b < d.batch && iy >= 0 && iy < d.Hin && c0 + ci < d.Cin)
                    regU[i] = *reinterpret_cast<const uint4 *>(X + (long long)b * d.x_sb + (long long)(c0 + ci) * d.x_sc +
                                                               (long long)iy * d.x_sy + xg * VEC);
            }
        }
    };
    auto park = [&](int tile, int buf) {
        char *at = smem + buf * buf_bytes;
        T *raw = reinterpret_cast<T *>(at + a.a_bytes);
#pragma unroll
        for (int i = 0; i < A_PER; ++i) {
            const int c = tid + i * NT;
            if (c < A_CHUNKS) *reinterpret_cast<uint4 *>(at + (c / (KT / VEC)) * a.pitch_a + (c % (KT / VEC)) * 16) = regA[i];
        }
#pragma unroll
        for (int i = 0; i < U_MAX; ++i) {
            const int u = tid + i * NT;
            if (u < units) {
                const int row = fast_div(u, a.magic_xg), xg = u - row * a.xg;
                const int ci = fast_div(row, a.magic_rr), rr = row - ci * a.RR;
                u4raw w = {regU[i].x, regU[i].y, regU[i].z, regU[i].w};
                *reinterpret_cast<u4_unaligned *>(raw + ci * a.PLANE + rr * a.TW + d.padL + xg * VEC) = w;
            }
        }
        if (tid < GROUPS) {
            const int n0 = tile * KT;
            const int b0 = n0 / PP, y0 = (n0 - b0 * PP) / d.Wo;
            const int g0 = b0 * a.THP + y0 * d.sh;
            int p = n0 + tid * VEC, off = 0;
            if (p < a.N) {
                const int b = p / PP, rem = p - b * PP, y = rem / d.Wo, x = rem - y * d.Wo;
                off = (b * a.THP + y * d.sh - g0) * a.TW + x;
            }
            pixoff[buf][tid] = off;
        }
    };

    int buf = 0;
    if ((int)blockIdx.x < a.tiles) fetch(blockIdx.x);
    for (int tile = blockIdx.x; tile < a.tiles; tile += gridDim.x, buf ^= 1) {
        park(tile, buf);
        __syncthreads();  // tile parked; every wave is done with the tile before the previous one (same buffer)
        if (tile + (int)gridDim.x < a.tiles) fetch(tile + gridDim.x);
        const char *at = smem + buf * buf_bytes;
        const T *raw = reinterpret_cast<const T *>(at + a.a_bytes);
        for (int ks = wk; ks < KSTEPS; ks += 2) {
            const int po = pixoff[buf][ks * 2 + kg];
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

    // the two pixel-group halves meet in LDS, then one fp32 partial per workgroup
    float *red = reinterpret_cast<float *>(smem);
    constexpr int PER = RB * CBW * 16;
    if (wk == 1) {
        float *dst = red + (size_t)wc * PER * 64 + lane;
#pragma unroll
        for (int r = 0; r < RB; ++r)
#pragma unroll
            for (int jj = 0; jj < CBW; ++jj)
#pragma unroll
                for (int v = 0; v < 16; ++v) dst[((r * CBW + jj) * 16 + v) * 64] = acc[r][jj][v];
    }
    __syncthreads();
    if (wk == 0) {
        const float *src = red + (size_t)wc * PER * 64 + lane;
        const int Kw = d.Cin * taps;
        const int valid_cols = (d.Cin - c0 < a.CT ? d.Cin - c0 : a.CT) * taps;
        float *__restrict__ out = a.ws + (size_t)blockIdx.x * d.Cout * Kw + (size_t)c0 * taps;
#pragma unroll
        for (int r = 0; r < RB; ++r)
#pragma unroll
            for (int jj = 0; jj < CBW; ++jj) {
                const int m = (wc + 4 * jj) * 32 + lr;
                if (wc + 4 * jj >= a.cblocks || m >= valid_cols) continue;
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const int co = r0 + r * 32 + 8 * (v >> 2) + 4 * kg + (v & 3);
                    if (co < d.Cout) out[(size_t)co * Kw + m] = acc[r][jj][v] + src[((r * CBW + jj) * 16 + v) * 64];
                }
            }
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

template <typename T, int RB, int CBW>
static int launch_conv_wg(ConvWgArgs &a, int gy, int gz, void *dW, hipStream_t s) {
    constexpr int ES = (int)sizeof(T), VEC = 16 / ES;
    auto kern = conv_wg_kernel<T, RB, CBW>;
    a.pitch_a = 128 * ES + 16;
    a.a_bytes = 32 * RB * a.pitch_a;
    a.raw_bytes = (int)((((size_t)a.CT * a.PLANE * ES + 32) + 15) & ~(size_t)15);  // slack: a fragment may start at the last element
    const size_t red = (size_t)4 * RB * CBW * 16 * 64 * 4;
    if ((long)a.CT * a.RR * a.xg > 4L * 512) return -1;  // input units per thread that the prefetch registers hold
    size_t lds = 2 * ((size_t)a.a_bytes + a.raw_bytes);
    if (lds < red) lds = red;
    if (lds > 150 * 1024) return -1;
    static bool attr_set = false;
    if (!attr_set) {
        if (!hip_ok(hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, 150 * 1024),
                    "hipFuncSetAttribute"))
            return 2;
        attr_set = true;
    }
    // two workgroups per CU over the whole grid, each walking an equal share of the pixel tiles
    long parts = 2L * state().num_cu / ((long)gy * gz);
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
    a.N = d.batch * d.Ho * d.Wo;
    a.THP = d.Hin + d.padU + d.padD;
    a.TW = d.Win + d.padL + d.padR;
    if (d.padU < 0 || d.padD < 0 || d.padL < 0 || d.padR < 0) return -1;
    if ((d.Ho - 1) * d.sh + d.KH > a.THP || (d.Wo - 1) * d.sw + d.KW > a.TW) return -1;
    // 8 (4) consecutive pixels of a fragment must be 8 consecutive input columns of one row,
    // and input rows must be copyable 16 bytes at a time
    if (d.sw != 1 || d.Wo % VEC || d.Win % VEC || d.x_sy % VEC || d.x_sc % VEC || d.x_sb % VEC) return -1;
    if (reinterpret_cast<uintptr_t>(X) % 16 || reinterpret_cast<uintptr_t>(dY) % 16) return -1;
    a.tiles = (a.N + 127) / 128;
    // few pixel tiles: worth it only for small fp16 weight tensors (measured 8.6 against 11.2 us for one
    // 16->32 channel 32x32 sample, 14 against 9.5 us for eight 64->64 8x8 ones)
    if (st.gemm_path != 2 && a.tiles < st.num_cu && !(ES == 2 && (long)d.Cout * d.Cin * d.KH * d.KW <= 8192)) return -1;

    const int taps = d.KH * d.KW;
    a.RR = conv_raw_rows(128, d.Ho, d.Wo, d.sh, d.KH, a.THP, a.N);
    if (a.RR > 64) return -1;
    a.PLANE = a.RR * a.TW;
    a.CT = d.Cin <= 16 ? 16 : 32;
    a.xg = d.Win / VEC;
    if ((long)a.CT * a.RR * a.xg >= 65536 || (long)a.CT * taps >= 65536) return -1;
    a.cblocks = (a.CT * taps + 31) / 32;
    a.magic_xg = magic_of(a.xg);
    a.magic_rr = magic_of(a.RR);
    a.magic_taps = magic_of(taps);
    a.magic_kw = magic_of(d.KW);
    a.magic_thp = magic_of(a.THP);
    if (a.THP + a.RR >= 65536) return -1;
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
