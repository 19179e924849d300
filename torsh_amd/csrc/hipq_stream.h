// Streaming helpers shared by the calibration and special-scheme kernels: walk one or two f32
// arrays once with 16-byte loads (four in flight per lane on full tiles) and reduce across a
// wavefront.
#pragma once

#include "hipq_math.h"

namespace hipq {

constexpr int kCalBlock = 256;
constexpr int kCalVec = 4;                       // float4 loads in flight per lane
constexpr int kCalTile = kCalBlock * kCalVec;    // float4s per workgroup iteration

// Walks x[0..n) once: whole float4s through f4 (four loads in flight per lane on full tiles),
// the unaligned or ragged remainder through f1.
template <int BLOCK, typename F4, typename F1>
__device__ __forceinline__ void stream1(const float *__restrict__ x, size_t n, F4 f4, F1 f1) {
    constexpr int kTile = BLOCK * kCalVec;
    const bool aligned = (reinterpret_cast<uintptr_t>(x) & 15u) == 0;
    const size_t nvec = aligned ? n / 4 : 0;
    const float4 *x4 = reinterpret_cast<const float4 *>(x);
    const size_t ntiles = (nvec + kTile - 1) / kTile;
    for (size_t t = blockIdx.x; t < ntiles; t += gridDim.x) {
        const size_t base = t * kTile + threadIdx.x;
        if ((t + 1) * kTile <= nvec) {
            float4 v[kCalVec];
#pragma unroll
            for (int i = 0; i < kCalVec; ++i) v[i] = load_stream(x4 + base + size_t(i) * BLOCK);
#pragma unroll
            for (int i = 0; i < kCalVec; ++i) f4(v[i], base + size_t(i) * BLOCK);
        } else {
#pragma unroll
            for (int i = 0; i < kCalVec; ++i) {
                const size_t idx = base + size_t(i) * BLOCK;
                if (idx < nvec) f4(x4[idx], idx);
            }
        }
    }
    for (size_t i = nvec * 4 + size_t(blockIdx.x) * BLOCK + threadIdx.x; i < n; i += size_t(gridDim.x) * BLOCK)
        f1(x[i], i);
}

// Two inputs walked in step.
template <typename F4, typename F1>
__device__ __forceinline__ void stream2(const float *__restrict__ a, const float *__restrict__ b, size_t n, F4 f4,
                                        F1 f1) {
    const bool aligned = ((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b)) & 15u) == 0;
    const size_t nvec = aligned ? n / 4 : 0;
    const float4 *a4 = reinterpret_cast<const float4 *>(a);
    const float4 *b4 = reinterpret_cast<const float4 *>(b);
    constexpr int kHalf = kCalVec / 2;  // two loads per input in flight
    constexpr int kTile = kCalBlock * kHalf;
    const size_t ntiles = (nvec + kTile - 1) / kTile;
    for (size_t t = blockIdx.x; t < ntiles; t += gridDim.x) {
        const size_t base = t * kTile + threadIdx.x;
        if ((t + 1) * kTile <= nvec) {
            float4 va[kHalf], vb[kHalf];
#pragma unroll
            for (int i = 0; i < kHalf; ++i) {
                va[i] = load_stream(a4 + base + size_t(i) * kCalBlock);
                vb[i] = load_stream(b4 + base + size_t(i) * kCalBlock);
            }
#pragma unroll
            for (int i = 0; i < kHalf; ++i) f4(va[i], vb[i]);
        } else {
#pragma unroll
            for (int i = 0; i < kHalf; ++i) {
                const size_t idx = base + size_t(i) * kCalBlock;
                if (idx < nvec) f4(a4[idx], b4[idx]);
            }
        }
    }
    for (size_t i = nvec * 4 + size_t(blockIdx.x) * kCalBlock + threadIdx.x; i < n;
         i += size_t(gridDim.x) * kCalBlock)
        f1(a[i], b[i]);
}

__device__ __forceinline__ double wave_sum(double v) {
#pragma unroll
    for (int o = kWave / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
    return v;
}
__device__ __forceinline__ unsigned long long wave_sum(unsigned long long v) {
#pragma unroll
    for (int o = kWave / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
    return v;
}

}  // namespace hipq
