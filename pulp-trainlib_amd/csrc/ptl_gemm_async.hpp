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

}  // namespace ptl
