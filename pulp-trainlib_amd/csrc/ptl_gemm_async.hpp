// Declarations shared by the pipelined-GEMM translation units.
#pragma once
#include "ptl_common.hpp"

namespace ptl {

constexpr int ASYNC_KWMAX = 2048;  // k indices held in the kernel's look-up table

// One tile configuration of the pipelined kernel: BM x BN workgroup tile, NT
// threads, waves arranged WMv x WNv x WKv.  Defined (explicitly instantiated) in the
// ptl_gemm_async_<type>_c<n>.hip files.  Returns 0, 2 (HIP failure) or -1 (does
// not fit the LDS).
template <typename T, int BM, int BN, int NT, int WMv, int WNv, int WKv>
int launch_async(GemmArgs &g, const void *zero, hipStream_t s);

// Look-up-free loads need: no coordinates, a single-digit k axis with a
// non-negative stride, non-negative row offsets below 2^31 bytes, and a k range
// made of whole slabs (there is no zero fill on this path).
// Lean kernel for the case that both operands are plain (plain_operand() != 0).
template <typename T, int BM, int BN, int NT, int WMv, int WNv, int WKv, int NS, int G>
int launch_plain(GemmArgs &g, hipStream_t s);

template <typename T, int BM, int BN, int NT, int WMv, int WNv, int WKv, int NS, int G>
int launch_plain_pair(GemmArgs &g0, GemmArgs &g1, hipStream_t s);
template <typename T, int NS, int G>
int launch_plain_pair_mixed(GemmArgs &g0, GemmArgs &g1, hipStream_t s);

// Streaming kernel (A panel resident, column tiles streamed) for plain operands with K == KS slabs; -1 when
// the product does not fit it.
template <typename T, int BM, int BN, int KS>
int launch_stream(GemmArgs &g, int num_cu, hipStream_t s);

template <typename T>
inline int plain_operand(const OperandMap &om, int kchunk, int K) {
    constexpr int SK = 128 / (int)sizeof(T);
    if (om.mode != FILL_VEC_K && om.mode != FILL_VEC_R) return 0;
    const AxisMap &r = om.row, &k = om.k;
    bool nocoord = r.h2 == 0 && r.h1 == 0 && r.h0 == 0 && r.hb == 0 && r.w2 == 0 && r.w1 == 0 && r.w0 == 0 &&
                   r.wb == 0 && k.h2 == 0 && k.h1 == 0 && k.h0 == 0 && k.hb == 0 && k.w2 == 0 && k.w1 == 0 &&
                   k.w0 == 0 && k.wb == 0 && om.HL >= 1 && om.WL >= 1;
    if (!nocoord) return 0;
    if (!(k.d0 >= k.n) || k.o0 < 0 || k.ob < 0) return 0;
    if (r.o2 < 0 || r.o1 < 0 || r.o0 < 0 || r.ob < 0) return 0;
    if (K % SK != 0 || kchunk % SK != 0) return 0;
    // largest byte offset a thread can form: last row + one slab of k
    long long max_row = (long long)r.ob;
    int q0 = (r.d0 >= r.n ? r.n : r.d0) - 1, rest = r.d0 >= r.n ? 0 : (r.n - 1) / r.d0;
    int q1 = r.d1 >= (1 << 30) ? rest : (rest % r.d1), q2 = r.d1 >= (1 << 30) ? 0 : rest / r.d1;
    max_row += (long long)q0 * r.o0 + (long long)q1 * r.o1 + (long long)q2 * r.o2;
    long long max_off = (max_row + (long long)SK * k.o0) * (long long)sizeof(T);
    return max_off < ((long long)1 << 31) ? 1 : 0;
}
}  // namespace ptl
