// Shared helpers of the gfx950 kernels: element types, conversions, wave and
// block reductions, launch checking.  Everything here is device-inline or
// host-inline; each .hip file is a translation unit of its own.
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_bf16.h>
#include "infinicore_infer_hip.h"
#include <stdint.h>
#include <math.h>

#define IC_EXPORT extern "C" __attribute__((visibility("default")))

// Status codes of the C entry points.  0 = launched; hipError_t values are
// returned as they are (all positive); argument faults are negative.
#define IC_OK 0
#define IC_ERR_ARG (-1)
#define IC_ERR_UNSUPPORTED (-2)
#define IC_ERR_TOO_LARGE (-5)     // beyond the fixed capacity of an entry point that allocates nothing

// dtype codes shared with the Python binding.
#define IC_F32 0
#define IC_BF16 1

constexpr int kWave = 64;

typedef __hip_bfloat16 bf16;

// 16 bytes that this kernel reads once and nobody else soon (weights and cached keys and values streamed by a
// decode step): a load with the non-temporal hint, which the caches do not keep.  A kernel that only reads
// memory reaches 7.1 TB/s with it on MI355X against 6.0..6.3 TB/s with plain loads.  Not for operands that
// other blocks read again (token rows, keys and values of prompt tiles).
__device__ __forceinline__ uint4 load_stream16(const void* p) {
    typedef unsigned ic_v4u __attribute__((ext_vector_type(4)));
    const ic_v4u v = __builtin_nontemporal_load(reinterpret_cast<const ic_v4u*>(p));
    return uint4{v[0], v[1], v[2], v[3]};
}

__device__ __forceinline__ float to_f32(float v) { return v; }
__device__ __forceinline__ float to_f32(bf16 v) { return __bfloat162float(v); }

template <typename T> __device__ __forceinline__ T from_f32(float v);
template <> __device__ __forceinline__ float from_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ bf16 from_f32<bf16>(float v) { return __float2bfloat16(v); }  // nearest even

// bf16 <-> raw bits (for 16-byte vector loads)
__device__ __forceinline__ float bf16_bits_to_f32(uint16_t b) { return __uint_as_float(((uint32_t)b) << 16); }
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40);  // NaN stays NaN
    u += 0x7fffu + ((u >> 16) & 1u);                                          // round to nearest even
    return (uint16_t)(u >> 16);
}

// ---- reductions over a 64-lane wave ------------------------------------------
// up * silu(gate) with the hardware's exp2 and reciprocal (each good to an ulp): for results that are
// rounded to bfloat16.  The float32 path divides and calls expf.
__device__ __forceinline__ float silu_mul_fast(float g, float u) {
    return u * g * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * g));
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, kWave));
    return v;
}

// Sum over a whole block; every thread gets the result.  `red` is LDS of at
// least blockDim.x / 64 floats.  Safe to call repeatedly with the same `red`.
__device__ __forceinline__ float block_sum(float v, float* red) {
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
    v = wave_sum(v);
    __syncthreads();               // earlier readers of red are done
    if (lane == 0) red[w] = v;
    __syncthreads();
    float t = 0.f;
    for (int i = 0; i < nw; ++i) t += red[i];
    return t;
}
__device__ __forceinline__ float block_max(float v, float* red) {
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
    v = wave_max(v);
    __syncthreads();
    if (lane == 0) red[w] = v;
    __syncthreads();
    float t = red[0];
    for (int i = 1; i < nw; ++i) t = fmaxf(t, red[i]);
    return t;
}

static inline int ic_launch_status() {
    hipError_t e = hipGetLastError();
    return (int)e;
}
