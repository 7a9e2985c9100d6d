// Matrix products for 17..64 rows (decoding a few dozen requests, short prompt portions) whose
// result goes into the residual stream (the O and down projections, N = the model's width):
// P[s] = A[M, K_s] W[N, K_s]^T in float32 for S slices of K, and the kernel that sums the slices,
// adds them to the residual stream and applies the RMS norm that follows.
//
// Why slices of K: with 64 rows a block that owns 16 weight rows re-reads all of A (64 x K) from
// L2, several times the bytes of its weights, and a width of a few thousand makes too few blocks of
// any sensible size for 256 compute units.  Here a block owns 64 weight rows and one slice of K: A
// goes through LDS once per block (shared by its four waves), the weights stream straight from
// memory into operand layout, and (N / 64) x S blocks fill most of the chip.  The slices meet in
// the add + norm kernel, which runs after the library's product too.  Measured on MI355X with cold
// weights at 64 rows (this / the library, us): 2,304 x 2,304: 8.8 / 11.1; 2,304 x 5,760: 13.3 / 25.0.
// For wide results (QKV, gate/up: N of 7,000 and more) the library is faster and is used: every
// block re-reads its slice of A, N / 64 times the bytes of A in all, as much as the weights there.
//
// Block: 4 waves; wave w owns weight rows n0 + 16 w .. + 15 and all row tiles of A.  K advances in
// chunks of 128: the A chunk [16 MT rows, 128] lies in LDS (rows padded to 272 bytes: a wave's 16-byte
// reads then spread over all banks), the next chunk's A and W are in registers while this one
// multiplies.  v_mfma_f32_16x16x32_bf16 with the weights as first operand:
// D[i = 4 (l/16) + e][j = l % 16] = C[m = 16 mt + j][n = n0 + 16 w + i].
#include "common.h"
#include <type_traits>

namespace {

typedef short sk_v8s __attribute__((ext_vector_type(8)));
typedef __bf16 sk_v8b __attribute__((ext_vector_type(8)));
typedef float sk_v4f __attribute__((ext_vector_type(4)));

constexpr int kSkThreads = 256;
constexpr int kSkCols = 64;              // weight rows per block
constexpr int kSkChunk = 128;            // k per LDS stage
constexpr int kSkRowBytes = 2 * kSkChunk + 16;

__device__ __forceinline__ uint4 ld16(const uint16_t* p) { return *reinterpret_cast<const uint4*>(p); }

template <int MT>
__global__ void __launch_bounds__(kSkThreads)
gemm_splitk_kernel(const uint16_t* __restrict__ A, const uint16_t* __restrict__ W, float* __restrict__ P,
                   int M, int N, int K, int lda, int ldw, int chunks_per_slice, int rotate) {
    __shared__ __attribute__((aligned(16))) unsigned char a_lds[2][16 * MT][kSkRowBytes];
    // The weights come in whole cache lines, a wave's load covering 8 rows x 128 bytes with the non-temporal hint (a stream
    // of such loads runs a third faster than one of loads in operand layout, 16 rows x 64 bytes), and pass through
    // this wave-private tile on their way into operand layout (LDS serves a wave's requests in order: no barrier).
    __shared__ __attribute__((aligned(16))) unsigned char w_lds[kSkThreads / 64][16][kSkRowBytes];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r = lane & 15, kq = lane >> 4;
    const int n0 = blockIdx.x * kSkCols + 16 * wave;
    const int slice = blockIdx.y;
    const int n_chunks = (K + kSkChunk - 1) / kSkChunk;
    const int c_begin = slice * chunks_per_slice;
    const int c_end = (c_begin + chunks_per_slice < n_chunks) ? c_begin + chunks_per_slice : n_chunks;
    // Column blocks start their walk over the slice at different chunks and wrap around: blocks that run at the same
    // time then read different offsets inside the weight rows.  With rows a power of two apart (8 KB, 32 KB) the same
    // offset in every row falls into few memory channels, and all blocks walking in step queue up there: 4,096 x
    // 16,384 at 17..64 rows 36.7..38.6 -> 27.6..35.2 us; other shapes (rows of 4,608 bytes and the like) are unchanged.
    // The order of the sum differs from column block to column block but is fixed for each.
    const int c_len = c_end - c_begin;
    const int rot = (rotate && c_len > 0) ? (int)(blockIdx.x % (unsigned)c_len) : 0;
    auto k_of = [&](int c) {                        // first k of the chunk that is walked as number c
        int pc = c + rot;
        if (pc >= c_end) pc -= c_len;
        return (c < c_end ? pc : c_begin) * kSkChunk;
    };

    // this lane's weight row (clamped: rows beyond N repeat the last one and are not stored)
    // load i of a chunk: rows 8 (i % 2) + lane / 8 of the wave's 16, bytes 128 (i / 2) + 16 (lane % 8) of the chunk's 256
    const uint16_t* wp8[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        const int row = n0 + 8 * h + (lane >> 3);
        wp8[h] = W + (size_t)(row < N ? row : N - 1) * ldw + 8 * (lane & 7);
    }
    // the A pieces this thread brings into LDS: piece p = tid + 256 i is row p / 16, bytes 16 (p % 16) of the chunk
    const uint16_t* ap[MT];
    int a_row[MT], a_col[MT];
#pragma unroll
    for (int i = 0; i < MT; ++i) {
        const int p = tid + kSkThreads * i;
        a_row[i] = p >> 4;
        a_col[i] = (p & 15) * 8;
        const int m = (a_row[i] < M) ? a_row[i] : M - 1;
        ap[i] = A + (size_t)m * lda + a_col[i];
    }

    sk_v4f acc[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[mt] = sk_v4f{0.f, 0.f, 0.f, 0.f};

    // Four chunks are in flight per wave (four register sets taking turns, for the weights and for this thread's
    // pieces of A alike): the weights come from memory and a block has few waves, so the bytes in flight have to
    // come from depth; and since loads complete in the order they were issued, A must be asked for as far ahead
    // as the weights, or waiting for a fresh piece of A would wait for every older weight load too.  Iteration i
    // works on chunk c: it multiplies (weights from set c % 4, A from LDS stage c % 2), asks for chunk c + 4, and
    // moves the A of chunk c + 1 (asked for three iterations ago) into the other LDS stage.
    // Loads are unconditional, with addresses clamped into the row: a load inside a branch makes the compiler
    // wait for every load in flight where the branch joins.  What lies beyond K (or beyond the slice) must
    // count as zero: A is masked when it goes to LDS (its registers are read there anyway), so whatever the
    // clamped weight load brought is multiplied by zero.
    uint4 wreg[4][4], areg[4][MT];
    auto fetch_w = [&](int c, auto set) {
        constexpr int J = decltype(set)::value;
        const int k0 = k_of(c);
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int k = k0 + 64 * (u >> 1);
            const bool ok = c < c_end && k + 8 * (lane & 7) + 8 <= K;
            wreg[J][u] = load_stream16(wp8[u & 1] + (ok ? k : 0));
        }
    };
    auto fetch_a = [&](int c, auto set) {
        constexpr int J = decltype(set)::value;
        const int k0 = k_of(c);
#pragma unroll
        for (int i = 0; i < MT; ++i) {
            const bool ok = c < c_end && k0 + a_col[i] + 8 <= K;
            areg[J][i] = ld16(ap[i] + (ok ? k0 : -a_col[i]));
        }
    };
    auto stash = [&](int c, auto set) {            // chunk c, waiting in A register set `set`, into LDS stage set % 2
        constexpr int J = decltype(set)::value;
        const int k0 = k_of(c);
#pragma unroll
        for (int i = 0; i < MT; ++i) {
            const uint32_t m = (c < c_end && k0 + a_col[i] + 8 <= K) ? 0xffffffffu : 0u;
            const uint4 v = areg[J][i];
            *reinterpret_cast<uint4*>(&a_lds[J % 2][a_row[i]][2 * a_col[i]]) = uint4{v.x & m, v.y & m, v.z & m, v.w & m};
        }
    };
    auto multiply = [&](auto wset, auto stage) {
        constexpr int J = decltype(wset)::value, L = decltype(stage)::value;
#pragma unroll
        for (int u = 0; u < 4; ++u)
            *reinterpret_cast<uint4*>(&w_lds[wave][8 * (u & 1) + (lane >> 3)][128 * (u >> 1) + 16 * (lane & 7)]) = wreg[J][u];
        __builtin_amdgcn_wave_barrier();
        uint4 wop[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) wop[u] = *reinterpret_cast<const uint4*>(&w_lds[wave][r][64 * u + 16 * kq]);
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const sk_v8b w8 = __builtin_bit_cast(sk_v8b, wop[u]);
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                const uint4 a = *reinterpret_cast<const uint4*>(&a_lds[L][16 * mt + r][2 * (32 * u + 8 * kq)]);
                acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w8, __builtin_bit_cast(sk_v8b, a), acc[mt], 0, 0, 0);
            }
        }
    };
    using I0 = std::integral_constant<int, 0>;
    using I1 = std::integral_constant<int, 1>;
    using I2 = std::integral_constant<int, 2>;
    using I3 = std::integral_constant<int, 3>;
    // chunk c in register set `set` (its A already in LDS stage `stage`); `ahead`: chunks c + 4 and c + 5 may exist
    auto step = [&](int c, auto set, auto stage, auto next, auto ahead) {
        multiply(set, stage);
        if constexpr (decltype(ahead)::value) fetch_w(c + 4, set);
        __builtin_amdgcn_sched_barrier(0);
        stash(c + 1, next);                         // set `next` holds chunk c + 1; its LDS stage was last read before the previous barrier
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (decltype(ahead)::value) fetch_a(c + 5, next);      // the A registers of chunk c + 1 are free now
        __syncthreads();
    };
    fetch_w(c_begin, I0{});
    fetch_a(c_begin, I0{});
    fetch_w(c_begin + 1, I1{});                     // (beyond the slice these re-read the row's first piece: a cache hit)
    fetch_a(c_begin + 1, I1{});
    fetch_w(c_begin + 2, I2{});
    fetch_a(c_begin + 2, I2{});
    fetch_w(c_begin + 3, I3{});
    fetch_a(c_begin + 3, I3{});
    __builtin_amdgcn_sched_barrier(0);
    stash(c_begin, I0{});
    __builtin_amdgcn_sched_barrier(0);
    if (c_begin + 4 < c_end) fetch_a(c_begin + 4, I0{});
    __syncthreads();
    int c = c_begin;
    for (; c + 8 <= c_end; c += 4) {                // every chunk asked for here exists
        step(c, I0{}, I0{}, I1{}, std::true_type{});
        step(c + 1, I1{}, I1{}, I2{}, std::true_type{});
        step(c + 2, I2{}, I0{}, I3{}, std::true_type{});
        step(c + 3, I3{}, I1{}, I0{}, std::true_type{});
    }
    for (; c < c_end; c += 4) {                     // the last rounds ask for chunks only while there are any (a branch per load
        // group is fine here: nothing is in flight across it that a later wait would have to spare); chunks beyond
        // the slice multiply zeros
        if (c + 4 < c_end) { step(c, I0{}, I0{}, I1{}, std::true_type{}); } else { step(c, I0{}, I0{}, I1{}, std::false_type{}); }
        if (c + 5 < c_end) { step(c + 1, I1{}, I1{}, I2{}, std::true_type{}); } else { step(c + 1, I1{}, I1{}, I2{}, std::false_type{}); }
        if (c + 6 < c_end) { step(c + 2, I2{}, I0{}, I3{}, std::true_type{}); } else { step(c + 2, I2{}, I0{}, I3{}, std::false_type{}); }
        if (c + 7 < c_end) { step(c + 3, I3{}, I1{}, I0{}, std::true_type{}); } else { step(c + 3, I3{}, I1{}, I0{}, std::false_type{}); }
    }
    // P[slice][m][n]; rows of A beyond M and weight rows beyond N are dropped
    float* out = P + (size_t)slice * M * N;
    const int n = n0 + 4 * kq;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const int m = 16 * mt + r;
        if (m >= M) continue;
        float* o = out + (size_t)m * N + n;
        if (n + 4 <= N && (N & 3) == 0) *reinterpret_cast<float4*>(o) = make_float4(acc[mt][0], acc[mt][1], acc[mt][2], acc[mt][3]);
        else
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (n + e < N) o[e] = acc[mt][e];
    }
}

// sum of the S slices at (m, n .. n + 3), rounded to bfloat16 as the product would be when stored
__device__ __forceinline__ void sum4(const float* __restrict__ P, size_t slice_stride, int S, size_t at, float alpha, float* o) {
    float4 t = *reinterpret_cast<const float4*>(P + at);
    for (int s = 1; s < S; ++s) {
        const float4 v = *reinterpret_cast<const float4*>(P + s * slice_stride + at);
        t.x += v.x; t.y += v.y; t.z += v.z; t.w += v.w;
    }
    o[0] = bf16_bits_to_f32(f32_to_bf16_bits(alpha * t.x));
    o[1] = bf16_bits_to_f32(f32_to_bf16_bits(alpha * t.y));
    o[2] = bf16_bits_to_f32(f32_to_bf16_bits(alpha * t.z));
    o[3] = bf16_bits_to_f32(f32_to_bf16_bits(alpha * t.w));
}
// ---- after O and down: x += alpha * product; out = rmsnorm(x) * w ------------------------------------------
// One block a row, the row in registers between the sum of squares and the scaling (d % 4 == 0, d <= 16 * threads).
template <int VPT>
__global__ void splitk_add_norm_kernel(const float* __restrict__ P, int S, int M, float* __restrict__ x, float alpha,
                                       const float* __restrict__ w, uint16_t* __restrict__ out, int d, float eps) {
    __shared__ float red[16];
    const int m = blockIdx.x;
    const size_t ss = (size_t)M * d, row = (size_t)m * d;
    float v[VPT][4];
    float sq = 0.f;
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
        const int c = 4 * (threadIdx.x + i * blockDim.x);
        if (c < d) {
            float y[4];
            sum4(P, ss, S, row + c, 1.0f, y);
            const float4 xv = *reinterpret_cast<const float4*>(x + row + c);
            v[i][0] = xv.x + alpha * y[0]; v[i][1] = xv.y + alpha * y[1];
            v[i][2] = xv.z + alpha * y[2]; v[i][3] = xv.w + alpha * y[3];
            *reinterpret_cast<float4*>(x + row + c) = make_float4(v[i][0], v[i][1], v[i][2], v[i][3]);
#pragma unroll
            for (int e = 0; e < 4; ++e) sq += v[i][e] * v[i][e];
        }
    }
    sq = block_sum(sq, red);
    const float inv = 1.0f / sqrtf(sq / (float)d + eps);
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
        const int c = 4 * (threadIdx.x + i * blockDim.x);
        if (c < d) {
            const float4 wv = *reinterpret_cast<const float4*>(w + c);
            uint2 o;
            o.x = (uint32_t)f32_to_bf16_bits(v[i][0] * inv * wv.x) | ((uint32_t)f32_to_bf16_bits(v[i][1] * inv * wv.y) << 16);
            o.y = (uint32_t)f32_to_bf16_bits(v[i][2] * inv * wv.z) | ((uint32_t)f32_to_bf16_bits(v[i][3] * inv * wv.w) << 16);
            *reinterpret_cast<uint2*>(out + row + c) = o;
        }
    }
}

int compute_units_sk() {
    static int cus = 0;
    if (cus == 0) {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) == hipSuccess && hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0) cus = n;
        else cus = 256;
    }
    return cus;
}

bool splits_ok(const float* P, int S, int M, int N) {
    return P && S >= 1 && S <= 64 && M >= 1 && M <= 64 && N >= 1 && (((uintptr_t)P & 15) == 0) && ((size_t)M * N) % 4 == 0;
}

}  // namespace

// 1 when the sliced product takes these sizes: 1..64 rows of bfloat16, K a multiple of 8 and at least 64 (a lane's
// clamped load of a weight row's last chunk starts up to 56 elements into the row: shorter rows would be read past
// their end), aligned operands.
IC_EXPORT int ic_gemm_splitk_supported(int M, int N, int K, int lda, int ldw) {
    return M >= 1 && M <= 64 && N >= 1 && K >= 64 && K % 8 == 0 && lda % 8 == 0 && ldw % 8 == 0 && lda >= K && ldw >= K;
}

// Slices of K to use: blocks for about 7/8 of the compute units (beyond the units a second, part-filled round was
// slower, and every further slice is one more partial result to add), up to all of them where that makes a quarter more
// blocks (64 column blocks: 4 slices, 256 blocks, against 3 and 192; 8B shape, 17..64 rows: O 13.2..15.5 -> 11.4..13.5 us,
// down 37.9..44.1 -> 36.7..38.5), and never fewer than 4 chunks of 128 a slice (the depth of the loads in flight).
IC_EXPORT int ic_gemm_splitk_slices(int N, int K) {
    if (N <= 0 || K <= 0) return 1;
    const int col_blocks = (N + kSkCols - 1) / kSkCols, chunks = (K + kSkChunk - 1) / kSkChunk;
    const int cus = compute_units_sk();
    int want = (7 * cus / 8) / col_blocks;
    const int full = cus / col_blocks;
    if (4 * full >= 5 * want) want = full;
    want = want < 1 ? 1 : (want > 64 ? 64 : want);
    int per = (chunks + want - 1) / want;
    per = per < 4 ? 4 : per;
    const int s = (chunks + per - 1) / per;
    return s > 64 ? 64 : s;
}

// 1 when the sliced product is the faster way for this product: enough blocks to occupy half the chip.
// Up to 16 rows the few-row product with the residual add in its epilogue is the faster one, but for 13..16 rows of
// 16 KB and more (from 9 rows on it loads its token operand once per k-step: the 8B shape's down projection takes 34 us
// at 16 rows, the slices and the kernel that sums them 27.5; a decode step of that shape 4.06 -> 3.95 ms at batch 16,
// 3.76 -> 3.76 at 12, 3.64 -> 3.69 at 9).
IC_EXPORT int ic_gemm_splitk_pays(int M, int N, int K) {
    if (M <= 0 || M > 64 || N <= 0 || K <= 0 || N > 8192) return 0;
    if (M <= 16 && (M <= 12 || K < 8192)) return 0;
    const int col_blocks = (N + kSkCols - 1) / kSkCols;
    return 2 * col_blocks * ic_gemm_splitk_slices(N, K) >= compute_units_sk();
}

// P[s, m, n] (float32 [n_slices, M, N]) = A[m, K_s] . W[n, K_s] for the n_slices slices of K (whole chunks of 128).
IC_EXPORT int ic_gemm_splitk(const void* A, const void* W, float* P, int M, int N, int K, int lda, int ldw, int n_slices,
                             hipStream_t stream) {
    if (M <= 0 || N <= 0) return IC_OK;
    if (!A || !W || !P || !ic_gemm_splitk_supported(M, N, K, lda, ldw) || n_slices < 1 || n_slices > 64) return IC_ERR_ARG;
    if (((uintptr_t)A & 15) || ((uintptr_t)W & 15) || ((uintptr_t)P & 15)) return IC_ERR_ARG;
    const int chunks = (K + kSkChunk - 1) / kSkChunk, per = (chunks + n_slices - 1) / n_slices;
    if ((chunks + per - 1) / per != n_slices) return IC_ERR_ARG;      // a slice would be empty: ask ic_gemm_splitk_slices
    dim3 grid((N + kSkCols - 1) / kSkCols, n_slices), block(kSkThreads);
    const uint16_t* a = (const uint16_t*)A;
    const uint16_t* w = (const uint16_t*)W;
    if (M <= 16) hipLaunchKernelGGL(gemm_splitk_kernel<1>, grid, block, 0, stream, a, w, P, M, N, K, lda, ldw, per, 1);
    else if (M <= 32) hipLaunchKernelGGL(gemm_splitk_kernel<2>, grid, block, 0, stream, a, w, P, M, N, K, lda, ldw, per, 1);
    else if (M <= 48) hipLaunchKernelGGL(gemm_splitk_kernel<3>, grid, block, 0, stream, a, w, P, M, N, K, lda, ldw, per, 1);
    else hipLaunchKernelGGL(gemm_splitk_kernel<4>, grid, block, 0, stream, a, w, P, M, N, K, lda, ldw, per, 1);
    return ic_launch_status();
}

// x (float32 [M, d]) += alpha * (the product of slices P [S, M, d], rounded to bfloat16); out (bfloat16 [M, d]) = rmsnorm(x) * w.
IC_EXPORT int ic_splitk_add_rmsnorm(const float* P, int n_slices, int M, float* x, float alpha, const float* w, void* out, int d,
                                    float eps, hipStream_t stream) {
    if (M <= 0) return IC_OK;
    if (d <= 0 || !x || !w || !out || !splits_ok(P, n_slices, M, d)) return IC_ERR_ARG;
    if (((uintptr_t)x & 15) || ((uintptr_t)w & 15) || ((uintptr_t)out & 7)) return IC_ERR_ARG;
    if (d % 4) return IC_ERR_UNSUPPORTED;
    const int vecs = d / 4;
    int threads = ((vecs + 63) / 64) * 64;
    if (threads > 1024) threads = 1024;
    const int vpt = (vecs + threads - 1) / threads;
    if (vpt > 4) return IC_ERR_UNSUPPORTED;
    dim3 grid(M), block(threads);
    uint16_t* o = (uint16_t*)out;
    switch (vpt) {
    case 1: hipLaunchKernelGGL(splitk_add_norm_kernel<1>, grid, block, 0, stream, P, n_slices, M, x, alpha, w, o, d, eps); break;
    case 2: hipLaunchKernelGGL(splitk_add_norm_kernel<2>, grid, block, 0, stream, P, n_slices, M, x, alpha, w, o, d, eps); break;
    case 3: hipLaunchKernelGGL(splitk_add_norm_kernel<3>, grid, block, 0, stream, P, n_slices, M, x, alpha, w, o, d, eps); break;
    default: hipLaunchKernelGGL(splitk_add_norm_kernel<4>, grid, block, 0, stream, P, n_slices, M, x, alpha, w, o, d, eps); break;
    }
    return ic_launch_status();
}
