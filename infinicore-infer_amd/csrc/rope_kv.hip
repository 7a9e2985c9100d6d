// Rotary position encoding fused with the write of keys and values into the
// paged cache.  One pass over the fused projection output qkv[T, H]:
//   q heads: rotated in place,
//   k heads: rotated and stored to the token's cache slot,
//   v heads: copied to the token's cache slot.
// Pairs are (j, j + rot/2) of each head ("half-split"), the order the
// checkpoint's q_proj/k_proj rows are in.  cos/sin are float32 tables
// [max_pos, rot/2]; the rotation is done in float32.
//
// Cache layout of one layer: K and V planes [num_pages, n_kv_heads, page_size, head_dim].
#include "common.h"

template <typename T>
__global__ void rope_kv_kernel(T* __restrict__ qkv, const int* __restrict__ positions,
                               const float* __restrict__ cos_t, const float* __restrict__ sin_t,
                               T* __restrict__ kcache, T* __restrict__ vcache,
                               const int* __restrict__ slots,
                               int row_stride, int nh, int nkvh, int dh, int rot, int page_size) {
    const int t = blockIdx.x;
    T* row = qkv + (size_t)t * row_stride;
    const int pos = positions[t];
    const int half = rot >> 1;
    const float* cr = cos_t + (size_t)pos * half;
    const float* sr = sin_t + (size_t)pos * half;
    const int slot = (nkvh > 0) ? slots[t] : -1;
    const int pg = slot >= 0 ? slot / page_size : 0;
    const int off = slot >= 0 ? slot - pg * page_size : 0;

    // rotations of q and k heads
    const int n_rot = (nh + nkvh) * half;
    for (int i = threadIdx.x; i < n_rot; i += blockDim.x) {
        const int head = i / half, j = i - head * half;
        T* hp = row + (size_t)head * dh;
        const float a = to_f32(hp[j]), b = to_f32(hp[j + half]);
        const float c = cr[j], s = sr[j];
        const T ra = from_f32<T>(a * c - b * s);
        const T rb = from_f32<T>(a * s + b * c);
        if (head < nh) {
            hp[j] = ra;
            hp[j + half] = rb;
        } else if (slot >= 0) {
            T* kp = kcache + (((size_t)pg * nkvh + (head - nh)) * page_size + off) * dh;
            kp[j] = ra;
            kp[j + half] = rb;
        }
    }
    if (nkvh == 0 || slot < 0) return;
    // the part of each k head beyond the rotated dims passes through
    const int tail = dh - rot;
    if (tail > 0) {
        for (int i = threadIdx.x; i < nkvh * tail; i += blockDim.x) {
            const int kh = i / tail, j = rot + (i - kh * tail);
            kcache[(((size_t)pg * nkvh + kh) * page_size + off) * dh + j] = row[(size_t)(nh + kh) * dh + j];
        }
    }
    // values
    const T* vsrc = row + (size_t)(nh + nkvh) * dh;
    for (int i = threadIdx.x; i < nkvh * dh; i += blockDim.x) {
        const int kh = i / dh, j = i - kh * dh;
        vcache[(((size_t)pg * nkvh + kh) * page_size + off) * dh + j] = vsrc[i];
    }
}

// qkv: [T, row_stride] with q heads first, then (if nkvh > 0) k heads, then v heads.
// nkvh == 0: only q is rotated, nothing is written to the cache (a layer that
// reads another layer's cache).
IC_EXPORT int ic_rope_kv_write(void* qkv, int dtype, const int* positions, const float* cos_t,
                               const float* sin_t, void* kcache, void* vcache, const int* slots,
                               int T, int row_stride, int nh, int nkvh, int dh, int rot,
                               int page_size, hipStream_t stream) {
    if (T <= 0) return IC_OK;
    if (dh <= 0 || rot < 0 || rot > dh || (rot & 1) || nh < 0 || nkvh < 0 || page_size <= 0) return IC_ERR_ARG;
    if (row_stride < (nh + 2 * nkvh) * dh) return IC_ERR_ARG;
    dim3 grid(T), block(256);
    if (dtype == IC_F32)
        hipLaunchKernelGGL(rope_kv_kernel<float>, grid, block, 0, stream, (float*)qkv, positions, cos_t, sin_t,
                           (float*)kcache, (float*)vcache, slots, row_stride, nh, nkvh, dh, rot, page_size);
    else if (dtype == IC_BF16)
        hipLaunchKernelGGL(rope_kv_kernel<bf16>, grid, block, 0, stream, (bf16*)qkv, positions, cos_t, sin_t,
                           (bf16*)kcache, (bf16*)vcache, slots, row_stride, nh, nkvh, dh, rot, page_size);
    else
        return IC_ERR_UNSUPPORTED;
    return ic_launch_status();
}
