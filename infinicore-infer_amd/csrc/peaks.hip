// What the device can do at most, measured with kernels that do nothing else: the figures a kernel's share of
// "the peak" is priced against in the reports.  Not on the model's path.
//
// ic_peak_mfma_bf16: every wave issues v_mfma_f32_32x32x16_bf16 back to back on four independent accumulators
// (no loads, no LDS); the caller times the launch and divides the returned operation count by it.
// ic_peak_read: every block streams a contiguous share of a buffer with 16-byte loads that the caches do not keep
// (the non-temporal hint: 7.1 TB/s where plain loads reach 6.0..6.3), eight in flight per lane, and keeps a
// checksum so that the loads stay.
#include "common.h"

typedef __bf16 pk_bf16x8 __attribute__((ext_vector_type(8)));
typedef float pk_v16f __attribute__((ext_vector_type(16)));

__global__ void __launch_bounds__(256) peak_mfma_kernel(float* __restrict__ sink, int iters, float seed) {
    pk_bf16x8 a, b;
#pragma unroll
    for (int i = 0; i < 8; ++i) { a[i] = (__bf16)(seed + threadIdx.x * 0.001f + i); b[i] = (__bf16)(seed - i); }
    pk_v16f acc[4];
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[j][r] = 0.f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[j], 0, 0, 0);
    }
    float s = 0.f;
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) s += acc[j][r];
    if (s == 123456.789f) sink[0] = s;                       // never true in practice: the products stay
}

// Launches blocks_per_unit blocks of four waves per compute unit; returns the floating-point operations issued
// (2 per multiply-add), or a negative status.
IC_EXPORT long long ic_peak_mfma_bf16(float* sink, int iters, int blocks_per_unit, hipStream_t stream) {
    if (!sink || iters <= 0 || blocks_per_unit <= 0 || blocks_per_unit > 64) return IC_ERR_ARG;
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) return IC_ERR_ARG;
    const int blocks = cus * blocks_per_unit;
    hipLaunchKernelGGL(peak_mfma_kernel, dim3(blocks), dim3(256), 0, stream, sink, iters, 1.0f);
    const int st = ic_launch_status();
    if (st) return st;
    return (long long)blocks * 4 * iters * 4 * (2LL * 32 * 32 * 16);
}

__global__ void __launch_bounds__(256) peak_read_kernel(const uint4* __restrict__ src, long long n16, unsigned* __restrict__ sink) {
    const long long per = (n16 + gridDim.x - 1) / gridDim.x;
    const long long lo = (long long)blockIdx.x * per;
    long long hi = lo + per;
    if (hi > n16) hi = n16;
    unsigned s = 0;
    long long i = lo + threadIdx.x;
    for (; i + 7 * 256 < hi; i += 8 * 256) {
        uint4 v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = load_stream16(src + i + u * 256);
#pragma unroll
        for (int u = 0; u < 8; ++u) s += v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
    }
    for (; i < hi; i += 256) { const uint4 v = src[i]; s += v.x ^ v.y ^ v.z ^ v.w; }
    if (s == 0x9e3779b9u) sink[0] = s;                       // keeps the loads
}

// Reads `bytes` (a multiple of 16, 16-byte aligned) once.  0 or a negative status.
IC_EXPORT int ic_peak_read(const void* src, long long bytes, int blocks_per_unit, unsigned* sink, hipStream_t stream) {
    if (!src || !sink || bytes <= 0 || bytes % 16 || ((uintptr_t)src & 15) || blocks_per_unit <= 0 || blocks_per_unit > 64) return IC_ERR_ARG;
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) return IC_ERR_ARG;
    hipLaunchKernelGGL(peak_read_kernel, dim3(cus * blocks_per_unit), dim3(256), 0, stream, (const uint4*)src, bytes / 16, sink);
    return ic_launch_status();
}
