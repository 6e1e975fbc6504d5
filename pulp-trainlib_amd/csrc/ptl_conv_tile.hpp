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
