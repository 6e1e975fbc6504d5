// Pipelined GEMM, f16, 128x32 tile, 512 threads (waves 4x1x2): all sixteen operand fill-mode pairs.
#include "ptl_gemm_async.hpp"
#include "ptl_gemm_async.inc"

namespace ptl {
template int launch_async<ptl::half_t, 128, 32, 512, 4, 1, 2>(GemmArgs &, const void *, hipStream_t);
}
