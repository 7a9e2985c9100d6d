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

// ---- 16 bytes at a time ---------------------------------------------------------------------
template <typename T> struct Pack16;
template <> struct Pack16<float> {
    static constexpr int N = 4;
    __device__ static void load(const float* p, float* o) {
        const float4 v = *reinterpret_cast<const float4*>(p);
        o[0] = v.x; o[1] = v.y; o[2] = v.z; o[3] = v.w;
    }
    __device__ static void store(float* p, const float* o) {
        *reinterpret_cast<float4*>(p) = make_float4(o[0], o[1], o[2], o[3]);
    }
};
template <> struct Pack16<bf16> {
    static constexpr int N = 8;
    __device__ static void load(const bf16* p, float* o) {
        const uint4 v = *reinterpret_cast<const uint4*>(p);
        o[0] = __uint_as_float(v.x << 16); o[1] = __uint_as_float(v.x & 0xffff0000u);
        o[2] = __uint_as_float(v.y << 16); o[3] = __uint_as_float(v.y & 0xffff0000u);
        o[4] = __uint_as_float(v.z << 16); o[5] = __uint_as_float(v.z & 0xffff0000u);
        o[6] = __uint_as_float(v.w << 16); o[7] = __uint_as_float(v.w & 0xffff0000u);
    }
    __device__ static void store(bf16* p, const float* o) {
        uint4 v;
        v.x = (uint32_t)f32_to_bf16_bits(o[0]) | ((uint32_t)f32_to_bf16_bits(o[1]) << 16);
        v.y = (uint32_t)f32_to_bf16_bits(o[2]) | ((uint32_t)f32_to_bf16_bits(o[3]) << 16);
        v.z = (uint32_t)f32_to_bf16_bits(o[4]) | ((uint32_t)f32_to_bf16_bits(o[5]) << 16);
        v.w = (uint32_t)f32_to_bf16_bits(o[6]) | ((uint32_t)f32_to_bf16_bits(o[7]) << 16);
        *reinterpret_cast<uint4*>(p) = v;
    }
};

// The same work in 16-byte pieces.  Per token: (nh + nkvh) * (rot/2 / N) rotation items (N pairs
// each), nkvh * ((dh - rot) / N) pass-through items of k heads, nkvh * (dh / N) copy items of
// v heads.  Grid (T, ceil(items / 256)).  Needs rot/2, dh - rot and dh to be multiples of N.
template <typename T>
__global__ void __launch_bounds__(256)
rope_kv_vec_kernel(T* __restrict__ qkv, const int* __restrict__ positions,
                   const float* __restrict__ cos_t, const float* __restrict__ sin_t,
                   T* __restrict__ kcache, T* __restrict__ vcache, const int* __restrict__ slots,
                   int row_stride, int nh, int nkvh, int dh, int rot, int page_size) {
    constexpr int N = Pack16<T>::N;
    const int t = blockIdx.x;
    const int item = blockIdx.y * 256 + threadIdx.x;
    const int half = rot >> 1, cpr = half / N;                 // rotation items per head
    const int n_rot = (nh + nkvh) * cpr;
    const int cpt = (dh - rot) / N, n_tail = nkvh * cpt;       // pass-through items
    const int cpv = dh / N, n_v = nkvh * cpv;
    if (item >= n_rot + n_tail + n_v) return;
    T* row = qkv + (size_t)t * row_stride;
    size_t cbase = 0;                                          // element offset of kv head 0 of this token's slot
    bool have_slot = false;
    if (nkvh > 0) {
        const int slot = slots[t];
        have_slot = slot >= 0;
        const int pg = have_slot ? slot / page_size : 0, off = have_slot ? slot - pg * page_size : 0;
        cbase = ((size_t)pg * nkvh * page_size + off) * dh;
    }
    const size_t kv_head_stride = (size_t)page_size * dh;
    if (item < n_rot) {
        const int head = item / cpr, j = (item - head * cpr) * N;
        if (head >= nh && !have_slot) return;
        T* hp = row + (size_t)head * dh;
        const int pos = positions[t];
        float a[N], b[N], c[N], s[N], ra[N], rb[N];
        Pack16<T>::load(hp + j, a);
        Pack16<T>::load(hp + j + half, b);
#pragma unroll
        for (int e = 0; e < N; e += 4) {
            Pack16<float>::load(cos_t + (size_t)pos * half + j + e, c + e);
            Pack16<float>::load(sin_t + (size_t)pos * half + j + e, s + e);
        }
#pragma unroll
        for (int e = 0; e < N; ++e) { ra[e] = a[e] * c[e] - b[e] * s[e]; rb[e] = a[e] * s[e] + b[e] * c[e]; }
        T* o = (head < nh) ? hp : kcache + cbase + (size_t)(head - nh) * kv_head_stride;
        Pack16<T>::store(o + j, ra);
        Pack16<T>::store(o + j + half, rb);
        return;
    }
    if (!have_slot) return;
    float v[N];
    if (item < n_rot + n_tail) {
        const int i = item - n_rot, kh = i / cpt, j = rot + (i - kh * cpt) * N;
        Pack16<T>::load(row + (size_t)(nh + kh) * dh + j, v);
        Pack16<T>::store(kcache + cbase + (size_t)kh * kv_head_stride + j, v);
    } else {
        const int i = item - n_rot - n_tail, kh = i / cpv, j = (i - kh * cpv) * N;
        Pack16<T>::load(row + (size_t)(nh + nkvh + kh) * dh + j, v);
        Pack16<T>::store(vcache + cbase + (size_t)kh * kv_head_stride + j, v);
    }
}

template <typename T>
static bool launch_rope_vec(void* qkv, const int* positions, const float* cos_t, const float* sin_t,
                            void* kcache, void* vcache, const int* slots, int T_, int row_stride, int nh,
                            int nkvh, int dh, int rot, int page_size, hipStream_t stream) {
    constexpr int N = Pack16<T>::N;
    const int half = rot / 2;
    if (half % N || (dh - rot) % N || dh % N || row_stride % N || half % 4) return false;
    if (((uintptr_t)qkv & 15) || ((uintptr_t)kcache & 15) || ((uintptr_t)vcache & 15) ||
        ((uintptr_t)cos_t & 15) || ((uintptr_t)sin_t & 15)) return false;
    const int items = (nh + nkvh) * (half / N) + nkvh * ((dh - rot) / N) + nkvh * (dh / N);
    if (items <= 0 || (items + 255) / 256 > 65535) return false;
    dim3 grid(T_, (items + 255) / 256), block(256);
    hipLaunchKernelGGL(rope_kv_vec_kernel<T>, grid, block, 0, stream, (T*)qkv, positions, cos_t, sin_t,
                       (T*)kcache, (T*)vcache, slots, row_stride, nh, nkvh, dh, rot, page_size);
    return true;
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
    if (dtype == IC_F32 && launch_rope_vec<float>(qkv, positions, cos_t, sin_t, kcache, vcache, slots, T, row_stride, nh, nkvh, dh, rot, page_size, stream))
        return ic_launch_status();
    if (dtype == IC_BF16 && launch_rope_vec<bf16>(qkv, positions, cos_t, sin_t, kcache, vcache, slots, T, row_stride, nh, nkvh, dh, rot, page_size, stream))
        return ic_launch_status();
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
