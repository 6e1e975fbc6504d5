// A measurement aid, not part of the training path: what the matrix cores of this board sustain on a loop of
// nothing but fp16 MFMAs (no loads, no LDS), with operands that are random or all zero.  On random operands the
// board runs such a loop against its power limit and lowers its clock until the power fits; the rate it then holds
// is the ceiling that a GEMM or convolution kernel can approach on that data, whatever the published peak says.
#include "ptl_common.hpp"
#include "ptl_host.hpp"

namespace ptl {
namespace {

typedef _Float16 probe_f16x8 __attribute__((ext_vector_type(8)));
typedef float probe_f32x16 __attribute__((ext_vector_type(16)));
typedef float probe_f32x4 __attribute__((ext_vector_type(4)));

// SHAPE 32: v_mfma_f32_32x32x16_f16, eight accumulators; SHAPE 16: v_mfma_f32_16x16x32_f16, sixteen accumulators:
// 262144 flops per wave and iteration either way, no instruction waits for the one before it.
template <int SHAPE>
__global__ __launch_bounds__(512) void mfma_probe_kernel(const probe_f16x8 *__restrict__ src, float *__restrict__ out,
                                                         int iters) {
    const unsigned t = blockIdx.x * blockDim.x + threadIdx.x;
    probe_f16x8 a[4], b[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        a[i] = src[(t * 8 + i) & 0xFFFF];
        b[i] = src[(t * 8 + 4 + i) & 0xFFFF];
    }
    float s = 0.f;
    if constexpr (SHAPE == 32) {
        probe_f32x16 acc[8];
#pragma unroll
        for (int i = 0; i < 8; ++i)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][v] = 0.f;
        for (int it = 0; it < iters; ++it) {
#pragma unroll
            for (int i = 0; i < 8; ++i) acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[i & 3], b[i >> 1], acc[i], 0, 0, 0);
        }
#pragma unroll
        for (int i = 0; i < 8; ++i)
#pragma unroll
            for (int v = 0; v < 16; ++v) s += acc[i][v];
    } else {
        probe_f32x4 acc[16];
#pragma unroll
        for (int i = 0; i < 16; ++i)
#pragma unroll
            for (int v = 0; v < 4; ++v) acc[i][v] = 0.f;
        for (int it = 0; it < iters; ++it) {
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[i & 3], b[i >> 2], acc[i], 0, 0, 0);
        }
#pragma unroll
        for (int i = 0; i < 16; ++i)
#pragma unroll
            for (int v = 0; v < 4; ++v) s += acc[i][v];
    }
    out[t] = s;
}

__global__ __launch_bounds__(256) void probe_fill_kernel(unsigned *__restrict__ p, unsigned n, int random) {
    const unsigned i = blockIdx.x * 256u + threadIdx.x;
    if (i >= n) return;
    // two halves in (-0.5, 0.5) from an integer hash, or zeros
    unsigned h = i * 2654435761u;
    h ^= h >> 15;
    h *= 2246822519u;
    h ^= h >> 13;
    const _Float16 lo = (_Float16)(((h & 0xFFFF) / 65536.f) - 0.5f), hi = (_Float16)(((h >> 16) / 65536.f) - 0.5f);
    union {
        _Float16 e[2];
        unsigned u;
    } v;
    v.e[0] = lo;
    v.e[1] = hi;
    p[i] = random ? v.u : 0u;
}

}  // namespace
}  // namespace ptl

extern "C" int ptl_probe_mfma_fp16(int shape, int random_operands, int waves_per_simd, int iters, float *tflops) {
    using namespace ptl;
    if (!ensure_init()) return 2;
    if ((shape != 32 && shape != 16) || waves_per_simd < 1 || waves_per_simd > 2 || iters < 1 || !tflops) {
        set_error("ptl_probe_mfma_fp16: shape is 32 or 16, waves_per_simd 1 or 2, iters positive");
        return 1;
    }
    State &st = state();
    const int threads = 256 * waves_per_simd, blocks = st.num_cu;
    const size_t src_bytes = 65536 * 16, out_bytes = (size_t)blocks * threads * sizeof(float);
    char *buf = static_cast<char *>(scratch(src_bytes + out_bytes));
    if (!buf) return 2;
    hipLaunchKernelGGL(probe_fill_kernel, dim3((unsigned)(src_bytes / 4 / 256)), dim3(256), 0, st.stream,
                       reinterpret_cast<unsigned *>(buf), (unsigned)(src_bytes / 4), random_operands);
    auto launch = [&](int n) {
        if (shape == 32)
            hipLaunchKernelGGL((mfma_probe_kernel<32>), dim3(blocks), dim3(threads), 0, st.stream,
                               reinterpret_cast<const probe_f16x8 *>(buf), reinterpret_cast<float *>(buf + src_bytes), n);
        else
            hipLaunchKernelGGL((mfma_probe_kernel<16>), dim3(blocks), dim3(threads), 0, st.stream,
                               reinterpret_cast<const probe_f16x8 *>(buf), reinterpret_cast<float *>(buf + src_bytes), n);
    };
    launch(iters);  // warm-up: the clock settles under the load
    if (!hip_ok(hipEventRecord(st.ev0, st.stream), "hipEventRecord")) return 2;
    launch(iters);
    if (!hip_ok(hipEventRecord(st.ev1, st.stream), "hipEventRecord")) return 2;
    if (!hip_ok(hipEventSynchronize(st.ev1), "hipEventSynchronize")) return 2;
    float ms = 0.f;
    if (!hip_ok(hipEventElapsedTime(&ms, st.ev0, st.ev1), "hipEventElapsedTime")) return 2;
    const double flops = (double)blocks * (threads / 64) * (double)iters * 262144.0;
    *tflops = (float)(flops / (ms * 1e-3) / 1e12);
    return 0;
}
