// Lean pipelined GEMM for look-up-free operands, f16: the four tile configurations.
#include "ptl_gemm_async.hpp"
#include "ptl_gemm_plain.inc"

namespace ptl {
template int launch_plain<ptl::half_t, 128, 128, 512, 2, 2, 2, 3, 1>(GemmArgs &, hipStream_t);
template int launch_plain<ptl::half_t, 64, 64, 1024, 2, 2, 4, 3, 1>(GemmArgs &, hipStream_t);
template int launch_plain<ptl::half_t, 32, 128, 512, 1, 4, 2, 3, 1>(GemmArgs &, hipStream_t);
template int launch_plain<ptl::half_t, 128, 32, 512, 4, 1, 2, 3, 1>(GemmArgs &, hipStream_t);
template int launch_plain_pair<ptl::half_t, 128, 128, 512, 2, 2, 2, 3, 1>(GemmArgs &, GemmArgs &, hipStream_t);
template int launch_plain_pair<ptl::half_t, 64, 64, 1024, 2, 2, 4, 3, 1>(GemmArgs &, GemmArgs &, hipStream_t);
template int launch_plain_pair_mixed<ptl::half_t, 3, 1>(GemmArgs &, GemmArgs &, hipStream_t);
template int launch_plain<ptl::half_t, 64, 64, 1024, 2, 2, 4, 3, 2>(GemmArgs &, hipStream_t);
template int launch_plain<ptl::half_t, 128, 128, 256, 2, 2, 1, 2, 1>(GemmArgs &, hipStream_t);
template int launch_stream<ptl::half_t, 128, 64, 1>(GemmArgs &, int, hipStream_t);
template int launch_stream<ptl::half_t, 128, 64, 2>(GemmArgs &, int, hipStream_t);
template int launch_stream<ptl::half_t, 128, 64, 4>(GemmArgs &, int, hipStream_t);
template int launch_stream<ptl::half_t, 64, 64, 1>(GemmArgs &, int, hipStream_t);
template int launch_stream<ptl::half_t, 64, 64, 2>(GemmArgs &, int, hipStream_t);
template int launch_stream<ptl::half_t, 64, 64, 4>(GemmArgs &, int, hipStream_t);
template int launch_plain<ptl::half_t, 128, 64, 512, 2, 2, 2, 3, 1>(GemmArgs &, hipStream_t);
template int launch_plain<ptl::half_t, 256, 128, 512, 4, 2, 1, 3, 1>(GemmArgs &, hipStream_t);
template int launch_plain<ptl::half_t, 256, 256, 512, 2, 4, 1, 2, 1>(GemmArgs &, hipStream_t);
}
