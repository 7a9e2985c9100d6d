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

constexpr int kRopeHeadsPerBlock = 4;

// Grid (T, ceil((nh + 2 nkvh) / 4)), 256 threads: one wave per head of one token.
// Heads 0..nh-1 are q, then nkvh k heads, then nkvh v heads.
template <typename T>
__global__ void __launch_bounds__(64 * kRopeHeadsPerBlock)
rope_kv_kernel(T* __restrict__ qkv, const int* __restrict__ positions,
               const float* __restrict__ cos_t, const float* __restrict__ sin_t,
               T* __restrict__ kcache, T* __restrict__ vcache, const int* __restrict__ slots,
               int row_stride, int nh, int nkvh, int dh, int rot, int page_size) {
    const int t = blockIdx.x;
    const int head = blockIdx.y * kRopeHeadsPerBlock + (threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    if (head >= nh + 2 * nkvh) return;
    T* hp = qkv + (size_t)t * row_stride + (size_t)head * dh;
    const int half = rot >> 1;
    T* dst = nullptr;                       // where the head goes in the cache (k and v heads)
    if (head >= nh) {
        const int slot = slots[t];
        if (slot < 0) return;
        const int pg = slot / page_size, off = slot - pg * page_size;
        const int kh = (head < nh + nkvh) ? head - nh : head - nh - nkvh;
        T* plane = (head < nh + nkvh) ? kcache : vcache;
        dst = plane + (((size_t)pg * nkvh + kh) * page_size + off) * dh;
    }
    if (head >= nh + nkvh) {                // v: plain copy
        for (int j = lane; j < dh; j += 64) dst[j] = hp[j];
        return;
    }
    const int pos = positions[t];
    const float* cr = cos_t + (size_t)pos * half;
    const float* sr = sin_t + (size_t)pos * half;
    T* o = dst ? dst : hp;                  // q heads are rotated in place
    for (int j = lane; j < half; j += 64) {
        const float a = to_f32(hp[j]), b = to_f32(hp[j + half]);
        const float c = cr[j], s = sr[j];
        o[j] = from_f32<T>(a * c - b * s);
        o[j + half] = from_f32<T>(a * s + b * c);
    }
    if (dst)                                // the part of a k head beyond the rotated dims passes through
        for (int j = rot + lane; j < dh; j += 64) dst[j] = hp[j];
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
    if (T > 0x7fffffff || (nh + 2 * nkvh + kRopeHeadsPerBlock - 1) / kRopeHeadsPerBlock > 65535) return IC_ERR_ARG;
    dim3 grid(T, (nh + 2 * nkvh + kRopeHeadsPerBlock - 1) / kRopeHeadsPerBlock), block(64 * kRopeHeadsPerBlock);
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
