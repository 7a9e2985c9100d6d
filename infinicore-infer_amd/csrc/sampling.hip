// Sampling from float32 logits on the device: argmax, and temperature /
// top-k / top-p sampling with a caller-supplied uniform draw per row.
//
// One block of 1024 threads per row.  Every selection (the k-th largest logit, the
// probability at which the kept mass reaches top_p, the token at which the cumulated
// mass reaches the draw) is a radix select, 8 bits a pass, over an order-preserving
// integer image of the logit or over the token index.  Probability mass is summed in
// 40-bit fixed point with integer atomics, so no result depends on the order in which
// threads arrive.
//
// The row is walked as seldom as possible.  The first walk finds the maximum and counts
// the logits by the upper 12 bits of their image.  With a top-k that tells which few
// logits can matter (those in the k-th largest's bin and above): a second walk collects
// them (image and index) in LDS, and everything else works on that list.  With top-p
// alone a walk that sums the mass per bin comes between, and the list holds the bins
// down to the one in which the kept mass reaches top_p.  When the list would not fit
// (a flat distribution), or nothing is cut (temperature alone), the selections walk the
// whole row instead.
//
// Rules (the same as the plain implementation in the tests):
//   temperature == 0 or top_k == 1  -> argmax, lowest index among equals;
//   otherwise logits / temperature; keep every value >= the k-th largest
//   (k <= 0 or k >= V keeps all); w = exp(z - max); keep the most probable
//   tokens up to and including the one with which the kept mass reaches
//   top_p * total (equal values stay together); the token is the first, in
//   vocabulary order, whose cumulated kept mass reaches u * kept_total.
#include "common.h"
#include <atomic>
#include <mutex>

constexpr int kSampleThreads = 1024;
constexpr int kSampleWaves = kSampleThreads / 64;
constexpr int kBins = 4 * kSampleThreads;   // bins of the upper 12 bits of a logit's image; four a thread
constexpr int kBinShift = 20;
constexpr int kCand = 4096;                 // logits the list in LDS holds
static_assert(kBins == 1 << (32 - kBinShift), "a bin per value of the upper bits");
typedef unsigned long long u64;

__device__ __forceinline__ uint32_t order_key(float f) {
    const uint32_t u = __float_as_uint(f);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float key_value(uint32_t key) {     // the logit of an image
    return __uint_as_float((key & 0x80000000u) ? (key & 0x7fffffffu) : ~key);
}

__device__ __forceinline__ u64 fixed_mass(float x, float maxv, float inv_t) {
    const float w = expf((x - maxv) * inv_t);          // in (0, 1]
    return (u64)(w * 1099511627776.0f);                // 2^40
}

__device__ __forceinline__ u64 shfl_up_u64(u64 v, int o) {
    const uint32_t lo = __shfl_up((uint32_t)v, o, kWave), hi = __shfl_up((uint32_t)(v >> 32), o, kWave);
    return ((u64)hi << 32) | lo;
}

// f(x, i) for every logit of the row, four independent loads in flight per thread.
template <typename F>
__device__ __forceinline__ void for_each_logit(const float* __restrict__ row, int V, F f) {
    int i = threadIdx.x;
    for (; i + 3 * kSampleThreads < V; i += 4 * kSampleThreads) {
        const float x0 = row[i], x1 = row[i + kSampleThreads], x2 = row[i + 2 * kSampleThreads],
                    x3 = row[i + 3 * kSampleThreads];
        f(x0, i); f(x1, i + kSampleThreads); f(x2, i + 2 * kSampleThreads); f(x3, i + 3 * kSampleThreads);
    }
    for (; i < V; i += kSampleThreads) f(row[i], i);
}

// What the selections share in LDS.
struct SelectShared {
    u64 hist[256];
    u64 need;
    u64 above;
    int digit;
    int bin;
};

// Wave 0: the first of the 256 digits, walking down from 255 (DESC) or up from 0, at which the
// summed hist reaches need; what was still needed on entering it goes to sh.need.
template <bool DESC>
__device__ __forceinline__ void digit_select(SelectShared& sh, u64 need) {
    const int lane = threadIdx.x;
    u64 v[4], s = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int p = 4 * lane + j;
        v[j] = sh.hist[DESC ? 255 - p : p];
        s += v[j];
    }
    u64 incl = s;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
        const u64 t = shfl_up_u64(incl, o);
        if (lane >= o) incl += t;
    }
    u64 c = incl - s;
    if (lane == 63 && incl < need) { sh.digit = DESC ? 0 : 255; sh.need = 1; }   // cannot happen with need <= total
    if (c < need && need <= incl) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            if (c + v[j] >= need) {
                const int p = 4 * lane + j;
                sh.digit = DESC ? 255 - p : p;
                sh.need = need - c;
                break;
            }
            c += v[j];
        }
    }
}

// MODE 0: the largest image K with #{kept images >= K} >= need.
// MODE 1: the largest image K with mass{kept images >= K} >= need.
// MODE 2: the smallest index I with mass{kept, index <= I} >= need.
// kept: image >= min_key.  The elements come from the list in LDS (n of them) or, with LIST false, from the row.
template <int MODE, bool LIST>
__device__ uint32_t radix_select(const float* __restrict__ row, int V, const uint32_t* ckey, const int* cidx, int n,
                                 uint32_t min_key, u64 need, float maxv, float inv_t, SelectShared& sh) {
    uint32_t prefix = 0;
    for (int pass = 0; pass < 4; ++pass) {
        const int shift = 24 - 8 * pass;
        for (int i = threadIdx.x; i < 256; i += blockDim.x) sh.hist[i] = 0;
        __syncthreads();
        auto add = [&](uint32_t key, int idx) {
            if (key < min_key) return;
            const uint32_t sel = (MODE == 2) ? (uint32_t)idx : key;
            if (pass > 0 && (sel >> (shift + 8)) != (prefix >> (shift + 8))) return;
            const u64 wgt = (MODE == 0) ? 1ull : fixed_mass(key_value(key), maxv, inv_t);
            if (wgt) atomicAdd(&sh.hist[(sel >> shift) & 255u], wgt);
        };
        if (LIST) {
            for (int i = threadIdx.x; i < n; i += blockDim.x) add(ckey[i], cidx[i]);
        } else {
            for_each_logit(row, V, [&](float x, int i) { add(order_key(x), i); });
        }
        __syncthreads();
        if (threadIdx.x < 64) {
            if (MODE == 2) digit_select<false>(sh, need);
            else digit_select<true>(sh, need);
        }
        __syncthreads();
        prefix |= ((uint32_t)sh.digit) << shift;
        need = sh.need;
        __syncthreads();
    }
    return prefix;
}

// Sum over the block of one value per thread.
__device__ u64 block_sum_u64(u64 part, u64* sh_total) {
    if (threadIdx.x == 0) *sh_total = 0;
    __syncthreads();
    if (part) atomicAdd(sh_total, part);
    __syncthreads();
    const u64 tot = *sh_total;
    __syncthreads();
    return tot;
}

// Summed mass of the kept elements (image >= min_key) of the list.
__device__ u64 list_mass(const uint32_t* ckey, int n, uint32_t min_key, float maxv, float inv_t, u64* sh_total) {
    u64 part = 0;
    for (int i = threadIdx.x; i < n; i += blockDim.x)
        if (ckey[i] >= min_key) part += fixed_mass(key_value(ckey[i]), maxv, inv_t);
    return block_sum_u64(part, sh_total);
}

// DESC: the highest bin b with sum of val[b..] >= need; else the lowest bin b with sum of val[..b] >= need.
// Thread t owns bins 4t..4t+3.  sh.above = the sum beyond b on the side the walk came from.
template <bool DESC, typename TV>
__device__ int boundary_bin(const TV* val, u64 need, u64* scan, SelectShared& sh) {
    const int tid = threadIdx.x;
    u64 v[4], s = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) { v[j] = val[4 * tid + j]; s += v[j]; }
    scan[tid] = s;
    if (tid == 0) { sh.bin = DESC ? 0 : kBins - 1; sh.above = 0; }
    __syncthreads();
    for (int o = 1; o < kSampleThreads; o <<= 1) {           // inclusive scan from the side the walk starts
        u64 add = 0;
        if (DESC) { if (tid + o < kSampleThreads) add = scan[tid + o]; }
        else { if (tid >= o) add = scan[tid - o]; }
        __syncthreads();
        scan[tid] += add;
        __syncthreads();
    }
    const u64 incl = scan[tid];
    u64 c = incl - s;
    if (c < need && need <= incl) {
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) {
            const int j = DESC ? 3 - jj : jj;
            if (c + v[j] >= need) { sh.bin = 4 * tid + j; sh.above = c; break; }
            c += v[j];
        }
    }
    __syncthreads();
    return sh.bin;
}

// Summed mass of the kept logits of the row, and (runs != nullptr, V <= 64 * kBins) the same per run of 64
// consecutive logits: the walk's step j has wave w on the logits 1024 j + 64 w .. + 63, which is run 16 j + w.
__device__ u64 row_mass_by_runs(const float* __restrict__ row, int V, uint32_t min_key, float maxv, float inv_t,
                                u64* runs, u64* sh_total) {
    const int tid = threadIdx.x, lane = tid & 63;
    const int v_round = (V + kSampleThreads - 1) / kSampleThreads * kSampleThreads;
    u64 part = 0;
    for (int i0 = tid; i0 < v_round; i0 += 4 * kSampleThreads) {
        float x[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {                   // without condition: beyond the row the last logit again, not counted
            const int i = i0 + u * kSampleThreads;
            x[u] = row[i < V ? i : V - 1];
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int i = i0 + u * kSampleThreads;
            if (i - lane >= v_round) break;             // the same for the whole wave
            u64 m = (i < V && order_key(x[u]) >= min_key) ? fixed_mass(x[u], maxv, inv_t) : 0;
            part += m;
            if (runs) {
#pragma unroll
                for (int o = 32; o > 0; o >>= 1) {
                    const uint32_t lo = __shfl_xor((uint32_t)m, o, kWave), hi = __shfl_xor((uint32_t)(m >> 32), o, kWave);
                    m += ((u64)hi << 32) | lo;
                }
                if (lane == 0) runs[i >> 6] = m;
            }
        }
    }
    return block_sum_u64(part, sh_total);
}

__global__ void __launch_bounds__(kSampleThreads)
sample_kernel(const float* __restrict__ logits, long long row_stride, int V,
              const float* __restrict__ temperature, const int* __restrict__ top_k,
              const float* __restrict__ top_p, const float* __restrict__ uniform,
              int* __restrict__ out) {
    __shared__ float red[kSampleWaves];
    __shared__ int redi[kSampleWaves];
    __shared__ uint32_t counts[kBins];                 // logits per bin
    __shared__ u64 big[kBins];                         // mass per bin, later the list: kCand images, then kCand indices
    __shared__ u64 scan[kSampleThreads];
    __shared__ SelectShared sh;
    __shared__ u64 sh_total;
    __shared__ int sh_n;
    static_assert(sizeof(u64) * kBins >= (sizeof(uint32_t) + sizeof(int)) * kCand, "the list fits where the masses were");
    uint32_t* ckey = reinterpret_cast<uint32_t*>(big);
    int* cidx = reinterpret_cast<int*>(ckey + kCand);

    const int r = blockIdx.x, tid = threadIdx.x;
    const float* row = logits + (size_t)r * row_stride;
    const float temp = temperature ? temperature[r] : 0.f;
    const int k = top_k ? top_k[r] : 1;
    const float tp = top_p ? top_p[r] : 1.f;
    const bool greedy = temp == 0.f || k == 1;
    const bool cut_k = k > 0 && k < V, cut_p = tp < 1.0f;
    const bool binned = !greedy && (cut_k || cut_p);   // the bins are of use only when something is cut

    // ---- first walk: the maximum and its first index; logits per bin ----------------------------
    if (binned) {
#pragma unroll
        for (int j = 0; j < 4; ++j) counts[4 * tid + j] = 0;
        __syncthreads();
    }
    float best = -INFINITY;
    int besti = 0x7fffffff;
    if (binned) {
        for_each_logit(row, V, [&](float x, int i) {
            if (x > best || (x == best && i < besti)) { best = x; besti = i; }
            atomicAdd(&counts[order_key(x) >> kBinShift], 1u);
        });
    } else {
        for_each_logit(row, V, [&](float x, int i) {
            if (x > best || (x == best && i < besti)) { best = x; besti = i; }
        });
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
    for (int w = 1; w < kSampleWaves; ++w)
        if (red[w] > best || (red[w] == best && redi[w] < besti)) { best = red[w]; besti = redi[w]; }
    __syncthreads();
    if (greedy) {
        if (tid == 0) out[r] = besti;
        return;
    }
    const float inv_t = 1.0f / temp;
    const float maxv = best;

    // ---- which bins can matter, and whether their logits fit in the list --------------------------
    int n_list = -1;                                   // < 0: no list, the selections walk the row
    u64 total = 0;                                     // mass of everything kept so far
    if (cut_k) {
        const int b = boundary_bin<true>(counts, (u64)k, scan, sh);
        const u64 n = sh.above + counts[b];
        if (n <= (u64)kCand) n_list = b;               // (the bin for now)
    } else if (cut_p) {
#pragma unroll
        for (int j = 0; j < 4; ++j) big[4 * tid + j] = 0;
        __syncthreads();
        for_each_logit(row, V, [&](float x, int) {
            const u64 m = fixed_mass(x, maxv, inv_t);
            if (m) atomicAdd(&big[order_key(x) >> kBinShift], m);
        });
        __syncthreads();
        total = block_sum_u64(big[4 * tid] + big[4 * tid + 1] + big[4 * tid + 2] + big[4 * tid + 3], &sh_total);
        u64 need = (u64)ceil((double)(tp > 0.f ? tp : 0.f) * (double)total);
        if (need < 1) need = 1;
        if (need > total) need = total;
        const int b = boundary_bin<true>(big, need, scan, sh);
        u64 mine = 0;
#pragma unroll
        for (int j = 0; j < 4; ++j)
            if (4 * tid + j >= b) mine += counts[4 * tid + j];
        const u64 n = block_sum_u64(mine, &sh_total);
        if (n <= (u64)kCand) n_list = b;
    }
    __syncthreads();
    if (n_list >= 0) {                                 // second (third) walk: collect the bins from n_list on
        const uint32_t from = (uint32_t)n_list;
        if (tid == 0) sh_n = 0;
        __syncthreads();
        for_each_logit(row, V, [&](float x, int i) {
            const uint32_t key = order_key(x);
            if ((key >> kBinShift) >= from) {
                const int slot = atomicAdd(&sh_n, 1);
                if (slot < kCand) { ckey[slot] = key; cidx[slot] = i; }
            }
        });
        __syncthreads();
        n_list = sh_n < kCand ? sh_n : kCand;
        __syncthreads();
    }

    uint32_t min_key = 0;
    if (n_list >= 0) {
        // ---- everything on the list -------------------------------------------------------------
        if (cut_k) {
            min_key = radix_select<0, true>(row, V, ckey, cidx, n_list, 0u, (u64)k, maxv, inv_t, sh);
            total = list_mass(ckey, n_list, min_key, maxv, inv_t, &sh_total);
        }
        if (cut_p) {
            u64 need = (u64)ceil((double)(tp > 0.f ? tp : 0.f) * (double)total);
            if (need < 1) need = 1;
            if (need > total) need = total;
            const uint32_t pk = radix_select<1, true>(row, V, ckey, cidx, n_list, min_key, need, maxv, inv_t, sh);
            if (pk > min_key) min_key = pk;
            total = list_mass(ckey, n_list, min_key, maxv, inv_t, &sh_total);
        }
        u64 target = (u64)ceil((double)uniform[r] * (double)total);
        if (target < 1) target = 1;
        if (target > total) target = total;
        const uint32_t tok = radix_select<2, true>(row, V, ckey, cidx, n_list, min_key, target, maxv, inv_t, sh);
        if (tid == 0) out[r] = (int)tok;
        return;
    }

    // ---- the same on the whole row ------------------------------------------------------------------
    const bool by_runs = V <= 64 * kBins;              // the token's run of 64 from per-run masses, else by stretches
    if (cut_k) min_key = radix_select<0, false>(row, V, nullptr, nullptr, 0, 0u, (u64)k, maxv, inv_t, sh);
    if (cut_p) {
        if (cut_k) total = row_mass_by_runs(row, V, min_key, maxv, inv_t, nullptr, &sh_total);
        u64 need = (u64)ceil((double)(tp > 0.f ? tp : 0.f) * (double)total);
        if (need < 1) need = 1;
        if (need > total) need = total;
        const uint32_t pk = radix_select<1, false>(row, V, nullptr, nullptr, 0, min_key, need, maxv, inv_t, sh);
        if (pk > min_key) min_key = pk;
    }
    if (by_runs) {
#pragma unroll
        for (int j = 0; j < 4; ++j) big[4 * tid + j] = 0;
        __syncthreads();
    }
    total = row_mass_by_runs(row, V, min_key, maxv, inv_t, by_runs ? big : nullptr, &sh_total);
    u64 target = (u64)ceil((double)uniform[r] * (double)total);
    if (target < 1) target = 1;
    if (target > total) target = total;
    if (by_runs) {
        // the run in which the cumulated mass reaches the target, then its 64 logits on one wave
        const int q = boundary_bin<false>(big, target, scan, sh);
        const u64 before = sh.above;
        if (tid < 64) {
            const int i = 64 * q + tid;
            const float x = row[i < V ? i : V - 1];
            const u64 m = (i < V && order_key(x) >= min_key) ? fixed_mass(x, maxv, inv_t) : 0;
            u64 incl = m;
#pragma unroll
            for (int o = 1; o < 64; o <<= 1) {
                const u64 t = shfl_up_u64(incl, o);
                if (tid >= o) incl += t;
            }
            const u64 hit = __ballot(m > 0 && before + incl >= target);
            if (tid == 0) out[r] = hit ? 64 * q + __ffsll((long long)hit) - 1 : besti;    // (a hit there is: target <= total)
        }
        return;
    }
    // the token in vocabulary order: a contiguous stretch of the row per thread, a scan over the threads, and
    // the thread in whose stretch the target falls walks it again
    const int chunk = (V + kSampleThreads - 1) / kSampleThreads;
    const int lo = tid * chunk;
    const int hi = (lo + chunk < V) ? lo + chunk : V;
    u64 mine = 0;
    for (int i = lo; i < hi; ++i) {
        const float x = row[i];
        if (order_key(x) >= min_key) mine += fixed_mass(x, maxv, inv_t);
    }
    scan[tid] = mine;
    __syncthreads();
    for (int o = 1; o < kSampleThreads; o <<= 1) {           // inclusive scan
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

// ---- greedy choice for callers that cannot allocate ------------------------------------------
// The partial results of the two-stage argmax live in a file-scope device array instead of a
// buffer the caller brings: kArgmaxStaticRows rows x 64 chunks x (float value, int index) = 512 KB,
// held by every GPU the library runs on until the process ends.  In host code the array's name is
// only a stand-in; its device address is asked for once per device and kept.
constexpr int kArgmaxStaticRows = 1024;
constexpr int kMaxDevices = 64;
static __device__ __align__(256) unsigned char scratch[(size_t)kArgmaxStaticRows * kArgmaxChunks * (sizeof(float) + sizeof(int))];
static std::atomic<void*> g_scratch_ptr[kMaxDevices];
static std::mutex g_scratch_mutex;

// Device address of `scratch` on the current device (asked for at the first call on that device).
static int static_scratch(void** ptr) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= kMaxDevices) return IC_ERR_ARG;
    void* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (!p) {
        std::lock_guard<std::mutex> hold(g_scratch_mutex);
        p = g_scratch_ptr[dev].load(std::memory_order_relaxed);
        if (!p) {
            e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
            if (e != hipSuccess) return (int)e;
            if (!p) return (int)hipErrorInvalidSymbol;
            g_scratch_ptr[dev].store(p, std::memory_order_release);
        }
    }
    *ptr = p;
    return IC_OK;
}

IC_EXPORT int ic_argmax_static_max_rows() { return kArgmaxStaticRows; }

// ic_argmax with the library's own scratch memory: no allocation, here or in anything it calls.
// Every (row, chunk) cell the second stage reads is written by the first stage of the same call, so
// nothing has to be cleared between calls; calls that overlap on one GPU share the array and race.
IC_EXPORT int ic_argmax_static(const float* logits, long long row_stride, int n_rows, int V, int* out,
                               hipStream_t stream) {
    if (n_rows <= 0) return IC_OK;
    if (n_rows > kArgmaxStaticRows) return IC_ERR_TOO_LARGE;
    if (V <= 0 || row_stride < V || !logits || !out) return IC_ERR_ARG;
    void* base = nullptr;
    int st = static_scratch(&base);
    if (st) return st;
    float* pval = reinterpret_cast<float*>(base);
    int* pidx = reinterpret_cast<int*>(reinterpret_cast<unsigned char*>(base)
                                       + (size_t)kArgmaxStaticRows * kArgmaxChunks * sizeof(float));
    hipLaunchKernelGGL(argmax_partial_kernel, dim3(kArgmaxChunks, n_rows), dim3(256), 0, stream, logits,
                       row_stride, V, pval, pidx);
    st = ic_launch_status();
    if (st) return st;
    hipLaunchKernelGGL(argmax_final_kernel, dim3(n_rows), dim3(64), 0, stream, pval, pidx, out);
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
