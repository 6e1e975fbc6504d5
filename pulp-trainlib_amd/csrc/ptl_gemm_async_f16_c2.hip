// Pipelined GEMM, f16, 32x128 tile, 512 threads (waves 1x4x2): all sixteen operand fill-mode pairs.
#include "ptl_gemm_async.hpp"
#include "ptl_gemm_async.inc"

namespace ptl {
template int launch_async<ptl::half_t, 32, 128, 512, 1, 4, 2>(GemmArgs &, const void *, hipStream_t);
}
