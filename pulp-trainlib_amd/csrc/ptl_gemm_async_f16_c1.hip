// Pipelined GEMM, f16, 64x64 tile, 1024 threads (waves 2x2x4): all sixteen operand fill-mode pairs.
#include "ptl_gemm_async.hpp"
#include "ptl_gemm_async.inc"

namespace ptl {
template int launch_async<ptl::half_t, 64, 64, 1024, 2, 2, 4>(GemmArgs &, const void *, hipStream_t);
}
