// The batch normalisation's statistics from partial sums, the same way in every kernel that needs them (the
// normalisation's own second kernel and the convolutions that apply a normalisation while they load their input):
// results that depend on the statistics come out bit for bit the same whichever kernel formed them.
#pragma once
#include <hip/hip_runtime.h>

namespace ptl {

// Sums of channel `c` over its parts ([channel][part][4] floats, 16-byte aligned), by one wave: lane i adds parts
// i, i + 64, ... in that order (four loads in flight at a time; a part that is not there adds zeros), then the lanes'
// sums meet in a butterfly.  Every lane returns the totals.
__device__ __forceinline__ float4 norm_fold_wave(const float *__restrict__ part, int nparts, int c, int lane) {
    const float4 *src = reinterpret_cast<const float4 *>(part) + (size_t)c * nparts;
    float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int base = 0; base < nparts; base += 256) {
        float4 p[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int i = base + 64 * u + lane;
            p[u] = i < nparts ? src[i] : make_float4(0.f, 0.f, 0.f, 0.f);
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            v.x += p[u].x;
            v.y += p[u].y;
            v.z += p[u].z;
            v.w += p[u].w;
        }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        v.x += __shfl_xor(v.x, off);
        v.y += __shfl_xor(v.y, off);
        v.z += __shfl_xor(v.z, off);
        v.w += __shfl_xor(v.w, off);
    }
    return v;
}

// The same sums (places 0 and 1 of a part) in two steps, for a kernel that wants the loads in the air before it issues
// the loads of its tile and the sums only behind them: channels c0 + wave + 16 r (r < R) of a 16-wave workgroup.  The
// first 256 parts (four per lane) are asked for early, the rest - batches of many hundred samples - is read when the
// sums are taken.  Bit for bit norm_fold_wave's sums.
template <int R>
struct NormFoldRegs {
    float2 v[R][4];
};
template <int R>
__device__ __forceinline__ void norm_fold_ask(NormFoldRegs<R> &f, const float *__restrict__ part, int nparts, int c0,
                                              int nch, int wave, int lane) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int c = wave + 16 * r;
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int i = 64 * u + lane;
            f.v[r][u] = make_float2(0.f, 0.f);
            if (c < nch && i < nparts) f.v[r][u] = *reinterpret_cast<const float2 *>(part + ((size_t)(c0 + c) * nparts + i) * 4);
        }
    }
}
template <int R>
__device__ __forceinline__ void norm_fold_take(const NormFoldRegs<R> &f, float2 (&t)[R], const float *__restrict__ part,
                                               int nparts, int c0, int nch, int wave, int lane) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
        t[r] = make_float2(0.f, 0.f);
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            t[r].x += f.v[r][u].x;
            t[r].y += f.v[r][u].y;
        }
        const int c = wave + 16 * r;
        if (nparts > 256 && c < nch)
            for (int i = 256 + lane; i < nparts; i += 64) {
                const float2 p = *reinterpret_cast<const float2 *>(part + ((size_t)(c0 + c) * nparts + i) * 4);
                t[r].x += p.x;
                t[r].y += p.y;
            }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            t[r].x += __shfl_xor(t[r].x, off);
            t[r].y += __shfl_xor(t[r].y, off);
        }
    }
}

// Mean and deviation the way the reference forms them (lib/sources/pulp_batchnorm_fp32.c:99-109: the variance as
// the mean of (x - mean)^2 expanded, eps added under the root).
__device__ inline void norm_mean_sd(float sum, float sum_sq, float count, float eps, float &mean, float &sd) {
    // (the fused operations spelled out: every kernel that calls this rounds at the same places)
    mean = sum / count;
    sd = sqrtf(fmaf(mean, mean, fmaf(-2.f * sum, mean, sum_sq) / count) + eps);
}

// One element of the forward pass, before the skip tensor, the ReLU and the rounding: the reference's
// ((x - mean) / sd) * w + b (lib/sources/pulp_batchnorm_fp32.c:109) with the division taken out of the loop
// (gain = w / sd, once per channel): the difference is kept first, so a mean that is large against the deviation
// costs nothing, and the result is within two roundings of the reference's.
__device__ inline float norm_forward(float x, float mean, float gain, float b) { return fmaf(x - mean, gain, b); }

}  // namespace ptl
