// Tile-shape and split selection of the pipelined GEMM.
#include "ptl_gemm_async.hpp"

namespace ptl {

// Pipelined GEMM.  Returns 0 on success, 2 on a HIP failure, -1 when the problem
// does not fit this kernel (caller falls back to the staged kernel).
// `g.a.mode` / `g.b.mode` must already be chosen; on success g.splits / g.ws say
// whether a split-K reduction has to follow.
template <typename T>
int gemm_async(GemmArgs &g) {
    State &st = state();
    st.last_gemm_streamed = 0;
    const void *zero = st.zeros;
    if (!zero) return -1;
    constexpr int SK = 128 / (int)sizeof(T);  // k elements per slab (128 bytes per row)
    // k = (outer, inner) with the inner digit contiguous in both operands and a whole number of slabs long
    // (the weight gradient of a pointwise layer over a batch: k = (sample, pixel)): the lean kernel walks it as
    // one flat axis whose slab pointers jump at the end of every inner run.
    bool runs = false;
    {
        auto two_digit = [](const AxisMap &k) {
            return k.d0 < k.n && k.d1 >= (1 << 30) && k.o0 == 1 && k.o1 >= k.d0 && k.ob >= 0 && k.h1 == 0 && k.h0 == 0 &&
                   k.hb == 0 && k.w1 == 0 && k.w0 == 0 && k.wb == 0;
        };
        const AxisMap &ka = g.a.k, &kb = g.b.k;
        if (g.taps <= 1 && g.a.mode == FILL_VEC_K && g.b.mode == FILL_VEC_K && two_digit(ka) && two_digit(kb) &&
            ka.d0 == kb.d0 && ka.d0 % SK == 0 && g.K % SK == 0) {
            GemmArgs flat = g;
            flat.a.k = axis_plain(g.K, 1, ka.ob);
            flat.b.k = axis_plain(g.K, 1, kb.ob);
            flat.seg_slabs = ka.d0 / SK;
            flat.a_seg_jump = ((long long)ka.o1 - ka.d0) * (long long)sizeof(T);
            flat.b_seg_jump = ((long long)kb.o1 - kb.d0) * (long long)sizeof(T);
            if (plain_operand<T>(flat.a, SK, g.K) && plain_operand<T>(flat.b, SK, g.K)) {
                g = flat;
                runs = true;
            }
        }
    }
    auto tiles = [&](int bm, int bn) { return (long)((g.N + bm - 1) / bm) * ((g.M + bn - 1) / bn); };
    int cfg;
    if (g.N <= 32)
        cfg = 2;
    else if (g.M <= 32)
        cfg = 3;
    else if (g.N <= 64 || g.M <= 64)  // a 128-wide tile would be half padding
        cfg = 1;
    else if (tiles(128, 128) >= st.num_cu)
        cfg = 0;
    else
        cfg = 1;
    long nt = cfg == 0 ? tiles(128, 128) : cfg == 1 ? tiles(64, 64) : cfg == 2 ? tiles(32, 128) : tiles(128, 32);
    // at most 64 columns and many rows (64 filters over a batch of pixels), or k in runs: a 128x64 tile halves
    // the reads of the narrow operand against 64x64 (+27 % measured on 64 -> 64 channels, 56x56, batch 128)
    // a long stream of k into a small output: bound by memory in fp16 (fewer, taller workgroups stream as fast
    // and leave fewer partial sums), by the MFMAs in fp32 (every CU needs its workgroup)
    const bool long_k = sizeof(T) == 2 && (runs || g.K >= 512 * SK);
    const bool tall = cfg == 1 && g.N >= 128 && g.M > 32 && (long_k || tiles(128, 64) >= 2L * st.num_cu);
    if (tall) nt = tiles(128, 64);

    g.splits = 1;
    g.kchunk = ((g.K + SK - 1) / SK) * SK;
    int want = 1;
    if (nt * 4 <= st.num_cu) want = (int)((st.num_cu + nt - 1) / nt);
    // a long stream of k is bound by memory, not by the number of workgroups: half as many splits stream
    // as fast and leave half as many partial sums to add
    if (long_k && want > 1) want = (want + 1) / 2;
    // Operands that are not on the look-up-free path index k through a table of ASYNC_KWMAX entries.
    const bool need_lut = !(plain_operand<T>(g.a, g.kchunk, g.K) && plain_operand<T>(g.b, g.kchunk, g.K));
    int need = need_lut ? (g.K + ASYNC_KWMAX - 1) / ASYNC_KWMAX : 1;
    if (want < need) want = need;
    if (g.taps > 1) {  // a sum over filter taps runs on the look-up-free kernel in one piece
        if (need_lut) return -1;
        want = 1;
    }
    if (want > 1) {
        int min_chunk = 4 * SK;
        int max_splits = (g.K + min_chunk - 1) / min_chunk;
        int sp = want < max_splits ? want : max_splits;
        if (sp > 1) {
            int chunk = (g.K + sp - 1) / sp;
            chunk = ((chunk + SK - 1) / SK) * SK;
            sp = (g.K + chunk - 1) / chunk;
            g.splits = sp;
            g.kchunk = chunk;
        }
    }
    if (g.kchunk > ASYNC_KWMAX &&
        !(plain_operand<T>(g.a, g.kchunk, g.K) && plain_operand<T>(g.b, g.kchunk, g.K)))
        return -1;
    if (g.splits > 1) {
        size_t bytes = (size_t)g.splits * g.N * g.M * sizeof(float);
        if (bytes > ((size_t)1 << 30)) return -1;
        g.ws = workspace(bytes);
        if (!g.ws) return 2;
    }
    if (plain_operand<T>(g.a, g.kchunk, g.K) && plain_operand<T>(g.b, g.kchunk, g.K)) {
        // few rows (or few columns: then the product is computed transposed, which changes nothing about its
        // sums), a shallow contraction and a long other side: resident panel, streamed tiles
        auto streams = [&](int few, int many) {
            return (few == 64 || few % 128 == 0) && few <= 256 && many % 64 == 0 &&
                   (long)(many / 64) * ((few + 127) / 128) >= 4L * st.num_cu;
        };
        if (g.splits == 1 && g.taps <= 1 && g.K % SK == 0 && g.K <= 4 * SK && (streams(g.N, g.M) || streams(g.M, g.N))) {
            GemmArgs gs = g;
            if (!streams(g.N, g.M)) {
                gs.A = g.B;
                gs.B = g.A;
                gs.a = g.b;
                gs.b = g.a;
                gs.N = g.M;
                gs.M = g.N;
                gs.c.n = g.c.m;
                gs.c.m = g.c.n;
            }
            const int ks = gs.K / SK;
            int rc = -1;
            if (gs.N == 64)
                rc = ks == 1   ? launch_stream<T, 64, 64, 1>(gs, st.num_cu, st.stream)
                     : ks == 2 ? launch_stream<T, 64, 64, 2>(gs, st.num_cu, st.stream)
                     : ks == 4 ? launch_stream<T, 64, 64, 4>(gs, st.num_cu, st.stream)
                               : -1;
            else
                rc = ks == 1   ? launch_stream<T, 128, 64, 1>(gs, st.num_cu, st.stream)
                     : ks == 2 ? launch_stream<T, 128, 64, 2>(gs, st.num_cu, st.stream)
                     : ks == 4 ? launch_stream<T, 128, 64, 4>(gs, st.num_cu, st.stream)
                               : -1;
            if (rc == 0) st.last_gemm_streamed = 1;
            if (rc != -1) return rc;
        }
        switch (cfg) {
            case 0:
                // one or two slabs deep (pointwise layers): four waves without a k split need half the
                // LDS for the parked tile, so two workgroups share a CU and overlap load, MFMA and store
                if (g.splits == 1 && g.K <= 2 * SK) return launch_plain<T, 128, 128, 256, 2, 2, 1, 2, 1>(g, st.stream);
                // fp16 products large enough to give every CU a larger tile.  Each of these tiles holds a CU by itself,
                // so a launch runs in rounds of num_cu workgroups; measured per round (4096^3 and 8192^2 x 4096): a
                // 256x128 workgroup takes 1.7 times as long as a 128x128 one and a 256x256 workgroup 1.8 times as
                // long as a 256x128 one, for two and four times the work.  The larger tiles move a third / half less
                // from L2 to LDS and read a quarter less LDS per MFMA (the LDS serves 128 bytes per clock, and fragment
                // reads alone keep it busy two thirds of the MFMA time on the 128x128 tile); they also pay where they
                // save a half-empty round (196 tall tiles in one round against 392 square ones in two).
                if constexpr (sizeof(T) == 2) {
                    const long r_big = (tiles(256, 256) + st.num_cu - 1) / st.num_cu;
                    const long r_tall = (tiles(256, 128) + st.num_cu - 1) / st.num_cu;
                    const long r_square = (tiles(128, 128) + st.num_cu - 1) / st.num_cu;
                    const long c_big = 306 * r_big, c_tall = 170 * r_tall, c_square = 100 * r_square;
                    if (g.splits == 1 && g.N >= 256 && g.M >= 256 && c_big < c_tall && c_big < c_square)
                        return launch_plain<T, 256, 256, 512, 2, 4, 1, 2, 1>(g, st.stream);
                    if (g.splits == 1 && g.N >= 256 && c_tall < c_square)
                        return launch_plain<T, 256, 128, 512, 4, 2, 1, 3, 1>(g, st.stream);
                }
                return launch_plain<T, 128, 128, 512, 2, 2, 2, 3, 1>(g, st.stream);
            case 1:
                // fp32 MFMAs are slow enough to matter at this size: when 64x64 tiles leave half the CUs
                // idle, 64x32 tiles put a workgroup on every CU
                // (fp16: measured no gain on 512 x 1024 x 1024, 15.96 against 16.2 us per step of three such products -
                // at that size a launch is its fixed latencies, not its MFMAs)
                if constexpr (sizeof(T) == 4) {
                    if (g.splits == 1 && tiles(64, 64) * 2 <= st.num_cu && g.M % 32 == 0)
                        return launch_plain<T, 64, 32, 512, 2, 1, 4, 3, 1>(g, st.stream);
                }
                if (tall) return launch_plain<T, 128, 64, 512, 2, 2, 2, 3, 1>(g, st.stream);
                // small tile: two slabs per wait-and-barrier when the slab count is even
                if (g.splits == 1 && (g.K / SK) % 2 == 0 && g.K >= 4 * SK) return launch_plain<T, 64, 64, 1024, 2, 2, 4, 3, 2>(g, st.stream);
                return launch_plain<T, 64, 64, 1024, 2, 2, 4, 3, 1>(g, st.stream);
            case 2: return launch_plain<T, 32, 128, 512, 1, 4, 2, 3, 1>(g, st.stream);
            default: return launch_plain<T, 128, 32, 512, 4, 1, 2, 3, 1>(g, st.stream);
        }
    }
    int rc = -1;
    switch (cfg) {
        case 0: rc = launch_async<T, 128, 128, 512, 2, 2, 2>(g, zero, st.stream); break;
        case 1: break;
        case 2: rc = launch_async<T, 32, 128, 512, 1, 4, 2>(g, zero, st.stream); break;
        default: rc = launch_async<T, 128, 32, 512, 4, 1, 2>(g, zero, st.stream); break;
    }
    // The small tile also takes the cases whose ring does not fit LDS with a larger one.
    if (rc == -1) rc = launch_async<T, 64, 64, 1024, 2, 2, 4>(g, zero, st.stream);
    return rc;
}

// Both products in one launch when they are look-up free, need no k split and agree on the
// tile shape; -1 otherwise (the caller then runs them one after the other).
template <typename T>
int gemm_async_pair(GemmArgs &g0, GemmArgs &g1) {
    State &st = state();
    constexpr int SK = 128 / (int)sizeof(T);
    GemmArgs *gs[2] = {&g0, &g1};
    int cfg[2];
    for (int i = 0; i < 2; ++i) {
        GemmArgs &g = *gs[i];
        g.splits = 1;
        g.kchunk = g.K;
        if (g.K % SK || !plain_operand<T>(g.a, g.kchunk, g.K) || !plain_operand<T>(g.b, g.kchunk, g.K)) return -1;
        auto tiles = [&](int bm, int bn) { return (long)((g.N + bm - 1) / bm) * ((g.M + bn - 1) / bn); };
        if (g.N <= 32 || g.M <= 32) return -1;
        cfg[i] = tiles(128, 128) >= st.num_cu ? 0 : 1;
        if (cfg[i] == 1 && tiles(64, 64) * 4 <= st.num_cu) return -1;  // would want a k split
    }
    if (cfg[0] != cfg[1]) return -1;
    if (cfg[0] == 0) return launch_plain_pair<T, 128, 128, 512, 2, 2, 2, 3, 1>(g0, g1, st.stream);
    // A first product with at most half the contraction of the second: tiles twice as large for it even the
    // workgroups out; taken where that brings the launch down to one workgroup per CU.
    auto tiles_of = [](const GemmArgs &g, int bm, int bn) { return (long)((g.N + bm - 1) / bm) * ((g.M + bn - 1) / bn); };
    if (g0.K * 2 <= g1.K && g0.N % 128 == 0 && tiles_of(g0, 64, 64) + tiles_of(g1, 64, 64) > st.num_cu &&
        tiles_of(g0, 128, 64) + tiles_of(g1, 64, 64) <= st.num_cu)
        return launch_plain_pair_mixed<T, 3, 1>(g0, g1, st.stream);
    return launch_plain_pair<T, 64, 64, 1024, 2, 2, 4, 3, 1>(g0, g1, st.stream);
}

template int gemm_async_pair<float>(GemmArgs &, GemmArgs &);
template int gemm_async_pair<half_t>(GemmArgs &, GemmArgs &);
template int gemm_async<float>(GemmArgs &);
template int gemm_async<half_t>(GemmArgs &);

}  // namespace ptl
