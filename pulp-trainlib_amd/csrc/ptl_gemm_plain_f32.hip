// Lean pipelined GEMM for look-up-free operands, f32: the four tile configurations.
#include "ptl_gemm_async.hpp"
#include "ptl_gemm_plain.inc"

namespace ptl {
template int launch_plain<float, 128, 128, 512, 2, 2, 2, 3, 1>(GemmArgs &, hipStream_t);
template int launch_plain<float, 64, 64, 1024, 2, 2, 4, 3, 1>(GemmArgs &, hipStream_t);
template int launch_plain<float, 32, 128, 512, 1, 4, 2, 3, 1>(GemmArgs &, hipStream_t);
template int launch_plain<float, 128, 32, 512, 4, 1, 2, 3, 1>(GemmArgs &, hipStream_t);
template int launch_plain_pair<float, 128, 128, 512, 2, 2, 2, 3, 1>(GemmArgs &, GemmArgs &, hipStream_t);
template int launch_plain_pair<float, 64, 64, 1024, 2, 2, 4, 3, 1>(GemmArgs &, GemmArgs &, hipStream_t);
template int launch_plain_pair_mixed<float, 3, 1>(GemmArgs &, GemmArgs &, hipStream_t);
template int launch_plain<float, 64, 64, 1024, 2, 2, 4, 3, 2>(GemmArgs &, hipStream_t);
template int launch_plain<float, 64, 32, 512, 2, 1, 4, 3, 1>(GemmArgs &, hipStream_t);
template int launch_plain<float, 128, 128, 256, 2, 2, 1, 2, 1>(GemmArgs &, hipStream_t);
template int launch_stream<float, 128, 64, 1>(GemmArgs &, int, hipStream_t);
template int launch_stream<float, 128, 64, 2>(GemmArgs &, int, hipStream_t);
template int launch_stream<float, 128, 64, 4>(GemmArgs &, int, hipStream_t);
template int launch_stream<float, 64, 64, 1>(GemmArgs &, int, hipStream_t);
template int launch_stream<float, 64, 64, 2>(GemmArgs &, int, hipStream_t);
template int launch_stream<float, 64, 64, 4>(GemmArgs &, int, hipStream_t);
template int launch_plain<float, 128, 64, 512, 2, 2, 2, 3, 1>(GemmArgs &, hipStream_t);
}
