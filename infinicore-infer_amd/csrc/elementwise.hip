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

IC_EXPORT int ic_swiglu(const void* gate_up, void* out, int dtype, int T, int di, hipStream_t stream) {
    if (T <= 0) return IC_OK;
    if (di <= 0) return IC_ERR_ARG;
    const size_t n = (size_t)T * di;
    int blocks = (int)((n + 255) / 256);
    if (blocks > 16384) blocks = 16384;
    if (dtype == IC_F32)
        hipLaunchKernelGGL(swiglu_kernel<float>, dim3(blocks), dim3(256), 0, stream, (const float*)gate_up, (float*)out, di, n);
    else if (dtype == IC_BF16)
        hipLaunchKernelGGL(swiglu_kernel<bf16>, dim3(blocks), dim3(256), 0, stream, (const bf16*)gate_up, (bf16*)out, di, n);
    else
        return IC_ERR_UNSUPPORTED;
    return ic_launch_status();
}
