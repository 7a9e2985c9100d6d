// Attention over the paged cache, general form: any head size that is a
// multiple of 8 elements, any number of heads and groups, any page size, an
// optional window, float32 or bfloat16 storage.  One wave per (token, head)
// walks the keys the token may see, 64 at a time, with a float32 running
// softmax.  It serves the float32 mode, head sizes the tiled kernels do not
// cover, and as the yardstick the tiled kernels are tested against.
//
// The token's own key and value are already in the cache when this runs.
#include "common.h"

constexpr int kMaxHeadDim = 512;

template <typename T>
__global__ void __launch_bounds__(64)
attn_generic_kernel(const T* __restrict__ q, int q_stride, T* __restrict__ out, int out_stride,
                    const T* __restrict__ kcache, const T* __restrict__ vcache,
                    const int* __restrict__ block_tables, int bt_stride,
                    const int* __restrict__ token_req, const int* __restrict__ positions,
                    int nh, int nkvh, int dh, int page_size, float scale, int window) {
    __shared__ float qs[kMaxHeadDim];
    __shared__ float ps[64];
    __shared__ long long vrow[64];

    const int h = blockIdx.x % nh, t = blockIdx.x / nh, lane = threadIdx.x;
    const int kvh = h / (nh / nkvh);
    const int pos = positions[t];
    const int* bt = block_tables + (size_t)token_req[t] * bt_stride;
    const T* qp = q + (size_t)t * q_stride + (size_t)h * dh;
    for (int d = lane; d < dh; d += 64) qs[d] = to_f32(qp[d]) * scale;
    __syncthreads();

    const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
    const int nd = (dh + 63) / 64;          // output dims per lane (<= 8)
    float acc[kMaxHeadDim / 64];
#pragma unroll
    for (int i = 0; i < kMaxHeadDim / 64; ++i) acc[i] = 0.f;
    float m = -INFINITY, l = 0.f;

    for (int kb = lo; kb <= pos; kb += 64) {
        const int key = kb + lane;
        const bool valid = key <= pos;
        float s = -INFINITY;
        long long base = 0;
        if (valid) {
            const int pg = bt[key / page_size];
            const int off = key % page_size;
            base = (((long long)pg * nkvh + kvh) * page_size + off) * dh;
            const T* kp = kcache + base;
            float dot = 0.f;
            for (int d = 0; d < dh; ++d) dot += qs[d] * to_f32(kp[d]);
            s = dot;
        }
        const float m_new = fmaxf(m, wave_max(s));       // lane 0 of every chunk is valid: m_new is finite
        const float p = valid ? expf(s - m_new) : 0.f;
        const float corr = expf(m - m_new);               // exp(-inf) = 0 on the first chunk
        l = l * corr + wave_sum(p);
        m = m_new;
        __syncthreads();
        ps[lane] = p;
        vrow[lane] = base;
        __syncthreads();
        const int nk = (pos - kb + 1 < 64) ? pos - kb + 1 : 64;
#pragma unroll
        for (int i = 0; i < kMaxHeadDim / 64; ++i) {
            if (i < nd) {
                const int d = lane + 64 * i;
                float a = acc[i] * corr;
                if (d < dh)
                    for (int kk = 0; kk < nk; ++kk) a += ps[kk] * to_f32(vcache[vrow[kk] + d]);
                acc[i] = a;
            }
        }
    }
    T* op = out + (size_t)t * out_stride + (size_t)h * dh;
    const float inv = 1.0f / l;
#pragma unroll
    for (int i = 0; i < kMaxHeadDim / 64; ++i) {
        const int d = lane + 64 * i;
        if (i < nd && d < dh) op[d] = from_f32<T>(acc[i] * inv);
    }
}

IC_EXPORT int ic_attn_generic(const void* q, int q_stride, void* out, int out_stride, int dtype,
                              const void* kcache, const void* vcache, const int* block_tables,
                              int bt_stride, const int* token_req, const int* positions, int T,
                              int nh, int nkvh, int dh, int page_size, float scale, int window,
                              hipStream_t stream) {
    if (T <= 0) return IC_OK;
    if (nh <= 0 || nkvh <= 0 || nh % nkvh || dh <= 0 || dh > kMaxHeadDim || page_size <= 0) return IC_ERR_ARG;
    if ((long long)T * nh > 0x7fffffffLL) return IC_ERR_ARG;
    dim3 grid((unsigned)(T * nh)), block(64);
    if (dtype == IC_F32)
        hipLaunchKernelGGL(attn_generic_kernel<float>, grid, block, 0, stream, (const float*)q, q_stride,
                           (float*)out, out_stride, (const float*)kcache, (const float*)vcache, block_tables,
                           bt_stride, token_req, positions, nh, nkvh, dh, page_size, scale, window);
    else if (dtype == IC_BF16)
        hipLaunchKernelGGL(attn_generic_kernel<bf16>, grid, block, 0, stream, (const bf16*)q, q_stride,
                           (bf16*)out, out_stride, (const bf16*)kcache, (const bf16*)vcache, block_tables,
                           bt_stride, token_req, positions, nh, nkvh, dh, page_size, scale, window);
    else
        return IC_ERR_UNSUPPORTED;
    return ic_launch_status();
}
