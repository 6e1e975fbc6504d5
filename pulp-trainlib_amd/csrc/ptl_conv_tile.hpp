// Direct (raw-tile) convolution for channel-major tensors: host interface.
#pragma once
#include "ptl_common.hpp"

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
};

// Launches the direct kernel; the output is written through `c` (n = pixel index over
// (sample, row, column), m = filter).  Returns 0, a positive status on a HIP error, or -1
// when the geometry does not fit the kernel (the caller then takes the GEMM route).
template <typename T>
int conv_tile(const ConvTileDesc &d, const void *X, const void *Wt, void *Y, const OutMap &c);

}  // namespace ptl

namespace ptl {

// Quotients by a divisor fixed per launch: magic = ceil(2^32 / d) gives exact n / d for
// n, d < 2^16; magic 0 stands for d == 1.
inline unsigned magic_of(int dv) { return dv <= 1 ? 0u : (unsigned)((((unsigned long long)1 << 32) + dv - 1) / dv); }
#if defined(__HIPCC__)
__device__ inline int fast_div(int n, unsigned magic) { return magic ? (int)__umulhi((unsigned)n, magic) : n; }
#endif

// Weight gradient of the same convolution:
//   dW(co, ci, ky, kx) = sum_{b, y, x} dY(b, co, y, x) * in(b, ci, y*sh + ky - padU, x*sw + kx - padL)
// with dY channel-major [b][Cout][Ho*Wo] and dW dense [Cout][Cin][KH][KW].  Returns 0, a positive
// status on a HIP error, or -1 when the geometry does not fit the kernel.
template <typename T>
int conv_tile_wg(const ConvTileDesc &d, const void *X, const void *dY, void *dW);

}  // namespace ptl
