// Sampling from float32 logits on the device: argmax, and temperature /
// top-k / top-p sampling with a caller-supplied uniform draw per row.
//
// One block of 1024 threads per row.  The selection steps (k-th largest
// logit, the probability at which the kept mass reaches top_p) are radix
// selects over an order-preserving integer image of the logit, 8 bits a pass.
// Probability mass is summed in 40-bit fixed point with integer atomics, so
// the result does not depend on the order in which threads arrive.
//
// Rules (the same as the plain implementation in the tests):
//   temperature == 0 or top_k == 1  -> argmax, lowest index among equals;
//   otherwise logits / temperature; keep every value >= the k-th largest
//   (k <= 0 or k >= V keeps all); w = exp(z - max); keep the most probable
//   tokens up to and including the one with which the kept mass reaches
//   top_p * total (equal values stay together); the token is the first, in
//   vocabulary order, whose cumulated kept mass reaches u * kept_total.
#include "common.h"

constexpr int kSampleThreads = 1024;
typedef unsigned long long u64;

__device__ __forceinline__ uint32_t order_key(float f) {
    const uint32_t u = __float_as_uint(f);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

__device__ __forceinline__ u64 fixed_mass(float x, float maxv, float inv_t) {
    const float w = expf((x - maxv) * inv_t);          // in (0, 1]
    return (u64)(w * 1099511627776.0f);                // 2^40
}

// Find the largest key K such that the summed weight of {kept elements with key >= K} >= need.
// weight = 1 (WEIGHTED == false) or the fixed-point mass.  All threads return K.
template <bool WEIGHTED>
__device__ uint32_t radix_select(const float* __restrict__ row, int V, uint32_t min_key, u64 need,
                                 float maxv, float inv_t, u64* hist, u64* sh_need, int* sh_digit) {
    uint32_t prefix = 0;
    for (int pass = 0; pass < 4; ++pass) {
        const int shift = 24 - 8 * pass;
        for (int i = threadIdx.x; i < 256; i += blockDim.x) hist[i] = 0;
        __syncthreads();
        for (int i = threadIdx.x; i < V; i += blockDim.x) {
            const float x = row[i];
            const uint32_t key = order_key(x);
            if (key < min_key) continue;
            if (pass > 0 && (key >> (shift + 8)) != (prefix >> (shift + 8))) continue;
            const u64 wgt = WEIGHTED ? fixed_mass(x, maxv, inv_t) : 1ull;
            if (wgt) atomicAdd(&hist[(key >> shift) & 255u], wgt);
        }
        __syncthreads();
        if (threadIdx.x == 0) {
            u64 cum = 0;
            int sel = 0;
            for (int dgt = 255; dgt >= 0; --dgt) {
                const u64 c = hist[dgt];
                if (cum + c >= need) { sel = dgt; break; }
                cum += c;
            }
            *sh_digit = sel;
            *sh_need = need - cum;
        }
        __syncthreads();
        prefix |= ((uint32_t)(*sh_digit)) << shift;
        need = *sh_need;
        __syncthreads();
    }
    return prefix;
}

__global__ void __launch_bounds__(kSampleThreads)
sample_kernel(const float* __restrict__ logits, long long row_stride, int V,
              const float* __restrict__ temperature, const int* __restrict__ top_k,
              const float* __restrict__ top_p, const float* __restrict__ uniform,
              int* __restrict__ out) {
    __shared__ float red[16];
    __shared__ int redi[16];
    __shared__ u64 hist[256];
    __shared__ u64 scan[kSampleThreads];
    __shared__ u64 sh_need;
    __shared__ int sh_digit;
    __shared__ u64 sh_total;

    const int r = blockIdx.x, tid = threadIdx.x;
    const float* row = logits + (size_t)r * row_stride;
    const float temp = temperature ? temperature[r] : 0.f;
    const int k = top_k ? top_k[r] : 1;
    const float tp = top_p ? top_p[r] : 1.f;

    // ---- max and its first index ------------------------------------------
    float best = -INFINITY;
    int besti = 0x7fffffff;
    for (int i = tid; i < V; i += blockDim.x) {
        const float x = row[i];
        if (x > best || (x == best && i < besti)) { best = x; besti = i; }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        const float ob = __shfl_xor(best, o, kWave);
        const int oi = __shfl_xor(besti, o, kWave);
        if (ob > best || (ob == best && oi < besti)) { best = ob; besti = oi; }
    }
    if ((tid & 63) == 0) { red[tid >> 6] = best; redi[tid >> 6] = besti; }
    __syncthreads();
    best = red[0]; besti = redi[0];
    for (int w = 1; w < (int)(blockDim.x >> 6); ++w)
        if (red[w] > best || (red[w] == best && redi[w] < besti)) { best = red[w]; besti = redi[w]; }
    __syncthreads();
    if (temp == 0.f || k == 1) {
        if (tid == 0) out[r] = besti;
        return;
    }
    const float inv_t = 1.0f / temp;
    const float maxv = best;

    // ---- top-k: smallest kept key -------------------------------------------
    uint32_t min_key = 0;
    if (k > 0 && k < V)
        min_key = radix_select<false>(row, V, 0u, (u64)k, maxv, inv_t, hist, &sh_need, &sh_digit);

    // ---- total mass of the kept set -------------------------------------------
    auto kept_mass = [&](uint32_t mk) -> u64 {
        u64 part = 0;
        for (int i = tid; i < V; i += blockDim.x) {
            const float x = row[i];
            if (order_key(x) >= mk) part += fixed_mass(x, maxv, inv_t);
        }
        if (tid == 0) sh_total = 0;
        __syncthreads();
        if (part) atomicAdd(&sh_total, part);
        __syncthreads();
        const u64 tot = sh_total;
        __syncthreads();
        return tot;
    };
    u64 total = kept_mass(min_key);

    // ---- top-p: raise the smallest kept key -----------------------------------
    if (tp < 1.0f) {
        double need_d = (double)(tp > 0.f ? tp : 0.f) * (double)total;
        u64 need = (u64)ceil(need_d);
        if (need < 1) need = 1;
        if (need > total) need = total;
        const uint32_t pk = radix_select<true>(row, V, min_key, need, maxv, inv_t, hist, &sh_need, &sh_digit);
        if (pk > min_key) min_key = pk;
        total = kept_mass(min_key);
    }

    // ---- inverse CDF in vocabulary order ----------------------------------------
    u64 target = (u64)ceil((double)uniform[r] * (double)total);
    if (target < 1) target = 1;
    if (target > total) target = total;
    const int chunk = (V + blockDim.x - 1) / blockDim.x;
    const int lo = tid * chunk;
    const int hi = (lo + chunk < V) ? lo + chunk : V;
    u64 mine = 0;
    for (int i = lo; i < hi; ++i) {
        const float x = row[i];
        if (order_key(x) >= min_key) mine += fixed_mass(x, maxv, inv_t);
    }
    scan[tid] = mine;
    __syncthreads();
    for (int o = 1; o < (int)blockDim.x; o <<= 1) {          // inclusive scan
        const u64 add = (tid >= o) ? scan[tid - o] : 0;
        __syncthreads();
        scan[tid] += add;
        __syncthreads();
    }
    const u64 incl = scan[tid], excl = incl - mine;
    if (mine > 0 && excl < target && target <= incl) {
        u64 c = excl;
        int tok = hi - 1;
        for (int i = lo; i < hi; ++i) {
            const float x = row[i];
            if (order_key(x) >= min_key) {
                c += fixed_mass(x, maxv, inv_t);
                if (c >= target) { tok = i; break; }
            }
        }
        out[r] = tok;
    }
}

// ---- argmax in two stages: many blocks per row, then one wave per row --------------------------
constexpr int kArgmaxChunks = 64;

__device__ __forceinline__ void argmax_merge(float& best, int& besti, float ob, int oi) {
    if (ob > best || (ob == best && oi < besti)) { best = ob; besti = oi; }
}

__global__ void __launch_bounds__(256)
argmax_partial_kernel(const float* __restrict__ logits, long long row_stride, int V,
                      float* __restrict__ pval, int* __restrict__ pidx) {
    __shared__ float red[4];
    __shared__ int redi[4];
    const int r = blockIdx.y, c = blockIdx.x, tid = threadIdx.x;
    const float* row = logits + (size_t)r * row_stride;
    const int per = (V + kArgmaxChunks - 1) / kArgmaxChunks;
    const int lo = c * per, hi = (lo + per < V) ? lo + per : V;
    float best = -INFINITY;
    int besti = 0x7fffffff;
    for (int i = lo + tid; i < hi; i += 256) argmax_merge(best, besti, row[i], i);
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) argmax_merge(best, besti, __shfl_xor(best, o, kWave), __shfl_xor(besti, o, kWave));
    if ((tid & 63) == 0) { red[tid >> 6] = best; redi[tid >> 6] = besti; }
    __syncthreads();
    if (tid == 0) {
        for (int w = 1; w < 4; ++w) argmax_merge(best, besti, red[w], redi[w]);
        pval[r * kArgmaxChunks + c] = best;
        pidx[r * kArgmaxChunks + c] = besti;
    }
}

__global__ void __launch_bounds__(64)
argmax_final_kernel(const float* __restrict__ pval, const int* __restrict__ pidx, int* __restrict__ out) {
    const int r = blockIdx.x, lane = threadIdx.x;
    float best = pval[r * kArgmaxChunks + lane];
    int besti = pidx[r * kArgmaxChunks + lane];
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) argmax_merge(best, besti, __shfl_xor(best, o, kWave), __shfl_xor(besti, o, kWave));
    if (lane == 0) out[r] = besti;
}

// Greedy choice for every row (lowest index among equal maxima).  scratch_val / scratch_idx:
// n_rows * 64 floats / ints.
IC_EXPORT int ic_argmax(const float* logits, long long row_stride, int n_rows, int V, float* scratch_val,
                        int* scratch_idx, int* out, hipStream_t stream) {
    if (n_rows <= 0) return IC_OK;
    if (V <= 0 || row_stride < V || n_rows > 65535) return IC_ERR_ARG;
    hipLaunchKernelGGL(argmax_partial_kernel, dim3(kArgmaxChunks, n_rows), dim3(256), 0, stream, logits,
                       row_stride, V, scratch_val, scratch_idx);
    int st = ic_launch_status();
    if (st) return st;
    hipLaunchKernelGGL(argmax_final_kernel, dim3(n_rows), dim3(64), 0, stream, scratch_val, scratch_idx, out);
    return ic_launch_status();
}

// logits [n_rows, V] float32 with row stride `row_stride` elements.  temperature,
// top_k, top_p, uniform: per-row device arrays; passing temperature == nullptr
// means argmax for every row.
IC_EXPORT int ic_sample(const float* logits, long long row_stride, int n_rows, int V,
                        const float* temperature, const int* top_k, const float* top_p,
                        const float* uniform, int* out, hipStream_t stream) {
    if (n_rows <= 0) return IC_OK;
    if (V <= 0 || row_stride < V) return IC_ERR_ARG;
    if (temperature && !uniform) return IC_ERR_ARG;
    hipLaunchKernelGGL(sample_kernel, dim3(n_rows), dim3(kSampleThreads), 0, stream, logits, row_stride, V,
                       temperature, top_k, top_p, uniform, out);
    return ic_launch_status();
}
