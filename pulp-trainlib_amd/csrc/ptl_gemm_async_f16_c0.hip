// Pipelined GEMM, f16, 128x128 tile, 512 threads (waves 2x2x2): all sixteen operand fill-mode pairs.
#include "ptl_gemm_async.hpp"
#include "ptl_gemm_async.inc"

namespace ptl {
template int launch_async<ptl::half_t, 128, 128, 512, 2, 2, 2>(GemmArgs &, const void *, hipStream_t);
}
