// Row-wise and element-wise kernels: embedding gather with scale, RMSNorm
// (alone, fused with the residual add, or on gathered rows), the residual add
// alone, and SwiGLU.  The residual stream is float32 in every mode; the other
// activations are float32 or bfloat16.  All arithmetic is float32.
#include "common.h"

// ---------------------------------------------------------------------------
// x[t, :] = table[tokens[t], :] * scale
// ---------------------------------------------------------------------------
template <typename TW>
__global__ void embed_kernel(const int* __restrict__ tokens, const TW* __restrict__ table,
                             float* __restrict__ x, int d, float scale) {
    const int t = blockIdx.x;
    const TW* row = table + (size_t)tokens[t] * d;
    float* o = x + (size_t)t * d;
    for (int i = threadIdx.x; i < d; i += blockDim.x) o[i] = to_f32(row[i]) * scale;
}

IC_EXPORT int ic_embed(const int* tokens, const void* table, int table_dtype, float* x,
                       int T, int d, float scale, hipStream_t stream) {
    if (T <= 0) return IC_OK;
    if (d <= 0) return IC_ERR_ARG;
    dim3 grid(T), block(256);
    if (table_dtype == IC_F32)
        hipLaunchKernelGGL(embed_kernel<float>, grid, block, 0, stream, tokens, (const float*)table, x, d, scale);
    else if (table_dtype == IC_BF16)
        hipLaunchKernelGGL(embed_kernel<bf16>, grid, block, 0, stream, tokens, (const bf16*)table, x, d, scale);
    else
        return IC_ERR_UNSUPPORTED;
    return ic_launch_status();
}

// ---- four elements at a time ----------------------------------------------------
__device__ __forceinline__ void load4(const float* p, float* o) {
    const float4 v = *reinterpret_cast<const float4*>(p);
    o[0] = v.x; o[1] = v.y; o[2] = v.z; o[3] = v.w;
}
__device__ __forceinline__ void load4(const bf16* p, float* o) {
    const uint2 v = *reinterpret_cast<const uint2*>(p);
    o[0] = __uint_as_float(v.x << 16); o[1] = __uint_as_float(v.x & 0xffff0000u);
    o[2] = __uint_as_float(v.y << 16); o[3] = __uint_as_float(v.y & 0xffff0000u);
}
__device__ __forceinline__ void store4(float* p, const float* o) {
    *reinterpret_cast<float4*>(p) = make_float4(o[0], o[1], o[2], o[3]);
}
__device__ __forceinline__ void store4(bf16* p, const float* o) {
    uint2 v;
    v.x = (uint32_t)f32_to_bf16_bits(o[0]) | ((uint32_t)f32_to_bf16_bits(o[1]) << 16);
    v.y = (uint32_t)f32_to_bf16_bits(o[2]) | ((uint32_t)f32_to_bf16_bits(o[3]) << 16);
    *reinterpret_cast<uint2*>(p) = v;
}

// One pass: a row lives in registers between the sum of squares and the scaling
// (d % 4 == 0, d <= 4 * VPT * blockDim).  ADD: x += alpha * y first, x written back.
template <typename TY, typename TO, int VPT, bool ADD>
__global__ void norm_row_kernel(float* __restrict__ x, const int* __restrict__ rows, const TY* __restrict__ y,
                                float alpha, const float* __restrict__ w, TO* __restrict__ out, int d,
                                float eps, float out_scale) {
    __shared__ float red[16];
    const int r = blockIdx.x;
    float* xr = x + (size_t)(rows ? rows[r] : r) * d;
    float v[VPT][4];
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
        const int c = 4 * (threadIdx.x + i * blockDim.x);
        if (c < d) {
            load4(xr + c, v[i]);
            if (ADD) {
                float yv[4];
                load4(y + (size_t)r * d + c, yv);
#pragma unroll
                for (int e = 0; e < 4; ++e) v[i][e] += alpha * yv[e];
                store4(xr + c, v[i]);
            }
#pragma unroll
            for (int e = 0; e < 4; ++e) ss += v[i][e] * v[i][e];
        }
    }
    ss = block_sum(ss, red);
    const float inv = 1.0f / sqrtf(ss / (float)d + eps);
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
        const int c = 4 * (threadIdx.x + i * blockDim.x);
        if (c < d) {
            float wv[4], o[4];
            load4(w + c, wv);
#pragma unroll
            for (int e = 0; e < 4; ++e) o[e] = v[i][e] * inv * wv[e] * out_scale;
            store4(out + (size_t)r * d + c, o);
        }
    }
}

// Threads per row and vectors per thread for the one-pass kernels; 0 if the row does not fit.
static inline int norm_row_shape(int d, int* threads) {
    if (d % 4) return 0;
    const int vecs = d / 4;
    int t = ((vecs + 63) / 64) * 64;
    if (t > 1024) t = 1024;
    *threads = t;
    const int vpt = (vecs + t - 1) / t;
    return vpt <= 4 ? vpt : 0;
}

template <typename TY, typename TO, bool ADD>
static bool launch_norm_row(float* x, const int* rows, const TY* y, float alpha, const float* w, TO* out,
                            int n_rows, int d, float eps, float out_scale, hipStream_t stream) {
    int threads = 0;
    const int vpt = norm_row_shape(d, &threads);
    if (!vpt || ((uintptr_t)x & 15) || ((uintptr_t)w & 15) || ((uintptr_t)out & 7) || (ADD && ((uintptr_t)y & 7)))
        return false;
    dim3 grid(n_rows), block(threads);
    switch (vpt) {
    case 1: hipLaunchKernelGGL((norm_row_kernel<TY, TO, 1, ADD>), grid, block, 0, stream, x, rows, y, alpha, w, out, d, eps, out_scale); break;
    case 2: hipLaunchKernelGGL((norm_row_kernel<TY, TO, 2, ADD>), grid, block, 0, stream, x, rows, y, alpha, w, out, d, eps, out_scale); break;
    case 3: hipLaunchKernelGGL((norm_row_kernel<TY, TO, 3, ADD>), grid, block, 0, stream, x, rows, y, alpha, w, out, d, eps, out_scale); break;
    default: hipLaunchKernelGGL((norm_row_kernel<TY, TO, 4, ADD>), grid, block, 0, stream, x, rows, y, alpha, w, out, d, eps, out_scale); break;
    }
    return true;
}

// ---------------------------------------------------------------------------
// out[r, :] = x[rows ? rows[r] : r, :] * rsqrt(mean(x^2) + eps) * w * out_scale
// ---------------------------------------------------------------------------
template <typename TO>
__global__ void rmsnorm_kernel(const float* __restrict__ x, const int* __restrict__ rows,
                               const float* __restrict__ w, TO* __restrict__ out, int d,
                               float eps, float out_scale) {
    __shared__ float red[16];
    const int r = blockIdx.x;
    const float* xr = x + (size_t)(rows ? rows[r] : r) * d;
    float ss = 0.f;
    for (int i = threadIdx.x; i < d; i += blockDim.x) { float v = xr[i]; ss += v * v; }
    ss = block_sum(ss, red);
    const float inv = 1.0f / sqrtf(ss / (float)d + eps);
    TO* o = out + (size_t)r * d;
    for (int i = threadIdx.x; i < d; i += blockDim.x)
        o[i] = from_f32<TO>(xr[i] * inv * w[i] * out_scale);
}

IC_EXPORT int ic_rmsnorm(const float* x, const int* rows, const float* w, void* out, int out_dtype,
                         int n_rows, int d, float eps, float out_scale, hipStream_t stream) {
    if (n_rows <= 0) return IC_OK;
    if (d <= 0) return IC_ERR_ARG;
    if (out_dtype == IC_F32 && launch_norm_row<float, float, false>((float*)x, rows, (const float*)nullptr, 0.f, w, (float*)out, n_rows, d, eps, out_scale, stream))
        return ic_launch_status();
    if (out_dtype == IC_BF16 && launch_norm_row<float, bf16, false>((float*)x, rows, (const float*)nullptr, 0.f, w, (bf16*)out, n_rows, d, eps, out_scale, stream))
        return ic_launch_status();
    dim3 grid(n_rows), block(d >= 1024 ? 256 : 128);
    if (out_dtype == IC_F32)
        hipLaunchKernelGGL(rmsnorm_kernel<float>, grid, block, 0, stream, x, rows, w, (float*)out, d, eps, out_scale);
    else if (out_dtype == IC_BF16)
        hipLaunchKernelGGL(rmsnorm_kernel<bf16>, grid, block, 0, stream, x, rows, w, (bf16*)out, d, eps, out_scale);
    else
        return IC_ERR_UNSUPPORTED;
    return ic_launch_status();
}

// ---------------------------------------------------------------------------
// x += alpha * y ;  out = rmsnorm(x) * w        (residual add fused with the next norm)
// ---------------------------------------------------------------------------
template <typename TY, typename TO>
__global__ void add_rmsnorm_kernel(float* __restrict__ x, const TY* __restrict__ y, float alpha,
                                   const float* __restrict__ w, TO* __restrict__ out, int d, float eps) {
    __shared__ float red[16];
    const int r = blockIdx.x;
    float* xr = x + (size_t)r * d;
    const TY* yr = y + (size_t)r * d;
    float ss = 0.f;
    for (int i = threadIdx.x; i < d; i += blockDim.x) {
        float v = xr[i] + alpha * to_f32(yr[i]);
        xr[i] = v;                       // read back below by the same thread
        ss += v * v;
    }
    ss = block_sum(ss, red);
    const float inv = 1.0f / sqrtf(ss / (float)d + eps);
    TO* o = out + (size_t)r * d;
    for (int i = threadIdx.x; i < d; i += blockDim.x) o[i] = from_f32<TO>(xr[i] * inv * w[i]);
}

IC_EXPORT int ic_add_rmsnorm(float* x, const void* y, int y_dtype, float alpha, const float* w,
                             void* out, int out_dtype, int T, int d, float eps, hipStream_t stream) {
    if (T <= 0) return IC_OK;
    if (d <= 0) return IC_ERR_ARG;
    bool done = false;
    if (y_dtype == IC_F32 && out_dtype == IC_F32) done = launch_norm_row<float, float, true>(x, nullptr, (const float*)y, alpha, w, (float*)out, T, d, eps, 1.f, stream);
    else if (y_dtype == IC_BF16 && out_dtype == IC_BF16) done = launch_norm_row<bf16, bf16, true>(x, nullptr, (const bf16*)y, alpha, w, (bf16*)out, T, d, eps, 1.f, stream);
    else if (y_dtype == IC_F32 && out_dtype == IC_BF16) done = launch_norm_row<float, bf16, true>(x, nullptr, (const float*)y, alpha, w, (bf16*)out, T, d, eps, 1.f, stream);
    else if (y_dtype == IC_BF16 && out_dtype == IC_F32) done = launch_norm_row<bf16, float, true>(x, nullptr, (const bf16*)y, alpha, w, (float*)out, T, d, eps, 1.f, stream);
    if (done) return ic_launch_status();
    dim3 grid(T), block(d >= 1024 ? 256 : 128);
    if (y_dtype == IC_F32 && out_dtype == IC_F32)
        hipLaunchKernelGGL((add_rmsnorm_kernel<float, float>), grid, block, 0, stream, x, (const float*)y, alpha, w, (float*)out, d, eps);
    else if (y_dtype == IC_BF16 && out_dtype == IC_BF16)
        hipLaunchKernelGGL((add_rmsnorm_kernel<bf16, bf16>), grid, block, 0, stream, x, (const bf16*)y, alpha, w, (bf16*)out, d, eps);
    else if (y_dtype == IC_F32 && out_dtype == IC_BF16)
        hipLaunchKernelGGL((add_rmsnorm_kernel<float, bf16>), grid, block, 0, stream, x, (const float*)y, alpha, w, (bf16*)out, d, eps);
    else if (y_dtype == IC_BF16 && out_dtype == IC_F32)
        hipLaunchKernelGGL((add_rmsnorm_kernel<bf16, float>), grid, block, 0, stream, x, (const bf16*)y, alpha, w, (float*)out, d, eps);
    else
        return IC_ERR_UNSUPPORTED;
    return ic_launch_status();
}

// ---------------------------------------------------------------------------
// x += alpha * y
// ---------------------------------------------------------------------------
template <typename TY>
__global__ void residual_add_kernel(float* __restrict__ x, const TY* __restrict__ y, float alpha, size_t n) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t step = (size_t)gridDim.x * blockDim.x;
    for (; i < n; i += step) x[i] += alpha * to_f32(y[i]);
}

IC_EXPORT int ic_residual_add(float* x, const void* y, int y_dtype, float alpha, long long n, hipStream_t stream) {
    if (n <= 0) return IC_OK;
    int blocks = (int)((n + 255) / 256);
    if (blocks > 8192) blocks = 8192;
    if (y_dtype == IC_F32)
        hipLaunchKernelGGL(residual_add_kernel<float>, dim3(blocks), dim3(256), 0, stream, x, (const float*)y, alpha, (size_t)n);
    else if (y_dtype == IC_BF16)
        hipLaunchKernelGGL(residual_add_kernel<bf16>, dim3(blocks), dim3(256), 0, stream, x, (const bf16*)y, alpha, (size_t)n);
    else
        return IC_ERR_UNSUPPORTED;
    return ic_launch_status();
}

// ---------------------------------------------------------------------------
// out[t, j] = up[t, j] * silu(gate[t, j]),  gate = gu[t, j], up = gu[t, di + j]
// ---------------------------------------------------------------------------
template <typename T>
__global__ void swiglu_kernel(const T* __restrict__ gu, T* __restrict__ out, int di, size_t n) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t step = (size_t)gridDim.x * blockDim.x;
    for (; i < n; i += step) {
        const size_t t = i / di;
        const int j = (int)(i - t * di);
        const float g = to_f32(gu[t * 2 * (size_t)di + j]);
        const float u = to_f32(gu[t * 2 * (size_t)di + di + j]);
        const float s = g / (1.0f + expf(-g));
        out[i] = from_f32<T>(u * s);
    }
}

// eight elements per thread (di % 8 == 0, 16-byte aligned rows)
__global__ void swiglu_vec8_kernel(const bf16* __restrict__ gu, bf16* __restrict__ out, int di, size_t n8) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t step = (size_t)gridDim.x * blockDim.x;
    const int per_row = di >> 3;
    for (; i < n8; i += step) {
        const size_t t = i / per_row;
        const int j = (int)(i - t * per_row) << 3;
        const bf16* gp = gu + t * 2 * (size_t)di + j;
        float g[8], u[8], o[8];
        load4(gp, g); load4(gp + 4, g + 4);
        load4(gp + di, u); load4(gp + di + 4, u + 4);
#pragma unroll
        for (int e = 0; e < 8; ++e) o[e] = silu_mul_fast(g[e], u[e]);
        bf16* op = out + t * (size_t)di + j;
        store4(op, o); store4(op + 4, o + 4);
    }
}

IC_EXPORT int ic_swiglu(const void* gate_up, void* out, int dtype, int T, int di, hipStream_t stream) {
    if (T <= 0) return IC_OK;
    if (di <= 0) return IC_ERR_ARG;
    const size_t n = (size_t)T * di;
    int blocks = (int)((n + 255) / 256);
    if (blocks > 16384) blocks = 16384;
    if (dtype == IC_BF16 && di % 8 == 0 && !((uintptr_t)gate_up & 15) && !((uintptr_t)out & 15)) {
        const size_t n8 = n / 8;
        int b8 = (int)((n8 + 255) / 256);
        if (b8 > 65536) b8 = 65536;
        hipLaunchKernelGGL(swiglu_vec8_kernel, dim3(b8), dim3(256), 0, stream, (const bf16*)gate_up, (bf16*)out, di, n8);
        return ic_launch_status();
    }
    if (dtype == IC_F32)
        hipLaunchKernelGGL(swiglu_kernel<float>, dim3(blocks), dim3(256), 0, stream, (const float*)gate_up, (float*)out, di, n);
    else if (dtype == IC_BF16)
        hipLaunchKernelGGL(swiglu_kernel<bf16>, dim3(blocks), dim3(256), 0, stream, (const bf16*)gate_up, (bf16*)out, di, n);
    else
        return IC_ERR_UNSUPPORTED;
    return ic_launch_status();
}


// ---------------------------------------------------------------------------
// Whole pages copied inside the planes of a cache group: for every plane p (a cache slot's keys or
// values) planes[p][dst[i]] = planes[p][src[i]].  Grid (pairs, planes); 16 bytes a thread and turn.
// ---------------------------------------------------------------------------
__global__ void __launch_bounds__(256)
copy_pages_kernel(uint4* __restrict__ planes, const int* __restrict__ src, const int* __restrict__ dst,
                  long long plane_vecs, long long page_vecs) {
    const uint4* from = planes + (size_t)blockIdx.y * plane_vecs + (size_t)src[blockIdx.x] * page_vecs;
    uint4* to = planes + (size_t)blockIdx.y * plane_vecs + (size_t)dst[blockIdx.x] * page_vecs;
    for (long long i = threadIdx.x; i < page_vecs; i += 256) to[i] = from[i];
}

// planes: n_planes planes of n_pages pages of page_bytes bytes each, one after the other.  src, dst: device int32 [n_pairs],
// page ids < n_pages; a page must not be both a source and a destination of one call.
IC_EXPORT int ic_copy_pages(void* planes, int n_planes, long long n_pages, long long page_bytes, const int* src, const int* dst,
                            int n_pairs, hipStream_t stream) {
    if (n_pairs <= 0 || n_planes <= 0) return IC_OK;
    if (!planes || !src || !dst || n_pages <= 0 || page_bytes <= 0 || page_bytes % 16 || ((uintptr_t)planes & 15) ||
        n_planes > 65535)
        return IC_ERR_ARG;
    hipLaunchKernelGGL(copy_pages_kernel, dim3(n_pairs, n_planes), dim3(256), 0, stream, (uint4*)planes, src, dst,
                       n_pages * (page_bytes / 16), page_bytes / 16);
    return ic_launch_status();
}
