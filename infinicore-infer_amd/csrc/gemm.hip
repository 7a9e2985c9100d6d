// C[M, N] = alpha * A[M, K] * W[N, K]^T for few rows M (decoding, the output
// head): bfloat16 operands on the matrix cores, float32 accumulation, float32
// or bfloat16 result.  The weight matrix is streamed once per 64 rows of A.
//
// Grid (ceil(N/16), ceil(M/(16*MT))), WPB waves.  Every wave owns the same
// 16 weight rows and a share of K (k-steps of 32, dealt in turn; WPB is 4, 8
// or 16 so that narrow matrices still fill the chip); lane
// (r = l%16, kq = l/16) loads 16 bytes W[n0+r][k0+8kq..+7] and the matching
// 16 bytes of each A row tile, and feeds them to two v_mfma_f32_16x16x16_bf16
// as A and B operands.  Both operands use the same lane->k mapping, so the
// order of k inside a step does not matter.  The waves' partial sums meet in LDS.
//
// 16x16x16 layout (lane l): A[i = l%16][k = 4(l/16)..+3], B[k = 4(l/16)..+3][j = l%16],
// D[i = 4(l/16) + e][j = l%16], e = 0..3.
#include "common.h"

typedef short v4s __attribute__((ext_vector_type(4)));
typedef float v4f __attribute__((ext_vector_type(4)));


// 8 consecutive bf16 from p (valid: how many of them exist), zero-filled.
template <bool ALIGNED>
__device__ __forceinline__ void load8(const uint16_t* __restrict__ p, int valid, v4s& lo, v4s& hi) {
    if (ALIGNED && valid >= 8) {
        const uint4 v = *reinterpret_cast<const uint4*>(p);
        lo[0] = (short)(v.x & 0xffff); lo[1] = (short)(v.x >> 16);
        lo[2] = (short)(v.y & 0xffff); lo[3] = (short)(v.y >> 16);
        hi[0] = (short)(v.z & 0xffff); hi[1] = (short)(v.z >> 16);
        hi[2] = (short)(v.w & 0xffff); hi[3] = (short)(v.w >> 16);
    } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            lo[e] = (e < valid) ? (short)p[e] : (short)0;
            hi[e] = (e + 4 < valid) ? (short)p[e + 4] : (short)0;
        }
    }
}

template <typename TC, int MT, int WPB, int UNROLL, bool ALIGNED>
__global__ void __launch_bounds__(WPB * 64)
gemm_nt_bf16_kernel(const uint16_t* __restrict__ A, const uint16_t* __restrict__ W, TC* __restrict__ C,
                    int M, int N, int K, int lda, int ldw, int ldc, float alpha) {
    __shared__ float red[WPB - 1][MT][64][4];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r = lane & 15, kq = lane >> 4;
    const int n0 = blockIdx.x * 16, m0 = blockIdx.y * (16 * MT);

    const int nrow = (n0 + r < N) ? n0 + r : N - 1;
    const uint16_t* wp = W + (size_t)nrow * ldw + 8 * kq;
    const uint16_t* ap[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const int mrow = (m0 + 16 * mt + r < M) ? m0 + 16 * mt + r : M - 1;
        ap[mt] = A + (size_t)mrow * lda + 8 * kq;
    }
    v4f acc[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[mt] = v4f{0.f, 0.f, 0.f, 0.f};

    // k-steps of 32 are dealt to the waves in turn; UNROLL steps are loaded before any is used
    const int nsteps = (K + 31) >> 5;
    for (int s0 = wave; s0 < nsteps; s0 += WPB * UNROLL) {
        v4s wlo[UNROLL], whi[UNROLL], alo[UNROLL][MT], ahi[UNROLL][MT];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            const int kk = 32 * (s0 + u * WPB);
            const int valid = K - kk - 8 * kq;          // <= 0 beyond the end of K
            if (valid > 0) load8<ALIGNED>(wp + kk, valid, wlo[u], whi[u]);
            else { wlo[u] = v4s{0, 0, 0, 0}; whi[u] = wlo[u]; }
        }
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            const int kk = 32 * (s0 + u * WPB);
            const int valid = K - kk - 8 * kq;
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                if (valid > 0) load8<ALIGNED>(ap[mt] + kk, valid, alo[u][mt], ahi[u][mt]);
                else { alo[u][mt] = v4s{0, 0, 0, 0}; ahi[u][mt] = alo[u][mt]; }
            }
        }
#pragma unroll
        for (int u = 0; u < UNROLL; ++u)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                acc[mt] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(wlo[u], alo[u][mt], acc[mt], 0, 0, 0);
                acc[mt] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(whi[u], ahi[u][mt], acc[mt], 0, 0, 0);
            }
    }
    if (wave > 0) {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int e = 0; e < 4; ++e) red[wave - 1][mt][lane][e] = acc[mt][e];
    }
    __syncthreads();
    if (wave > 0) return;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const int m = m0 + 16 * mt + r;             // column j of D = l % 16
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            float v = acc[mt][e];
#pragma unroll
            for (int w = 0; w < WPB - 1; ++w) v += red[w][mt][lane][e];
            const int n = n0 + 4 * kq + e;          // row i of D
            if (m < M && n < N) C[(size_t)m * ldc + n] = from_f32<TC>(alpha * v);
        }
    }
}

template <typename TC, int MT, int WPB, int UNROLL>
static void launch_gemm(const void* A, const void* W, void* C, int M, int N, int K, int lda, int ldw,
                        int ldc, float alpha, bool aligned, hipStream_t stream) {
    dim3 grid((N + 15) / 16, (M + 16 * MT - 1) / (16 * MT)), block(WPB * 64);
    if (aligned)
        hipLaunchKernelGGL((gemm_nt_bf16_kernel<TC, MT, WPB, UNROLL, true>), grid, block, 0, stream,
                           (const uint16_t*)A, (const uint16_t*)W, (TC*)C, M, N, K, lda, ldw, ldc, alpha);
    else
        hipLaunchKernelGGL((gemm_nt_bf16_kernel<TC, MT, WPB, UNROLL, false>), grid, block, 0, stream,
                           (const uint16_t*)A, (const uint16_t*)W, (TC*)C, M, N, K, lda, ldw, ldc, alpha);
}

// Waves per block: enough that row tiles x waves fill the chip's SIMDs a few times over.
template <typename TC>
static void dispatch_gemm(const void* A, const void* W, void* C, int M, int N, int K, int lda, int ldw,
                          int ldc, float alpha, bool aligned, hipStream_t stream) {
    const int tiles = (N + 15) / 16;
    if (M <= 16) {
        if (tiles < 256) launch_gemm<TC, 1, 16, 4>(A, W, C, M, N, K, lda, ldw, ldc, alpha, aligned, stream);
        else if (tiles < 600) launch_gemm<TC, 1, 8, 4>(A, W, C, M, N, K, lda, ldw, ldc, alpha, aligned, stream);
        else launch_gemm<TC, 1, 4, 4>(A, W, C, M, N, K, lda, ldw, ldc, alpha, aligned, stream);
    } else if (M <= 32) {
        if (tiles < 600) launch_gemm<TC, 2, 8, 4>(A, W, C, M, N, K, lda, ldw, ldc, alpha, aligned, stream);
        else launch_gemm<TC, 2, 4, 4>(A, W, C, M, N, K, lda, ldw, ldc, alpha, aligned, stream);
    } else {
        if (tiles < 600) launch_gemm<TC, 4, 8, 2>(A, W, C, M, N, K, lda, ldw, ldc, alpha, aligned, stream);
        else launch_gemm<TC, 4, 4, 2>(A, W, C, M, N, K, lda, ldw, ldc, alpha, aligned, stream);
    }
}

IC_EXPORT int ic_gemm_nt_supported(int a_dtype, int w_dtype, int c_dtype) {
    return a_dtype == IC_BF16 && w_dtype == IC_BF16 && (c_dtype == IC_F32 || c_dtype == IC_BF16);
}

IC_EXPORT int ic_gemm_nt(const void* A, int a_dtype, const void* W, int w_dtype, void* C, int c_dtype,
                         int M, int N, int K, int lda, int ldw, int ldc, float alpha, hipStream_t stream) {
    if (M <= 0 || N <= 0) return IC_OK;
    if (K <= 0 || lda < K || ldw < K || ldc < N) return IC_ERR_ARG;
    if (!ic_gemm_nt_supported(a_dtype, w_dtype, c_dtype)) return IC_ERR_UNSUPPORTED;
    if ((M + 63) / 64 > 65535) return IC_ERR_ARG;
    const bool aligned = (lda % 8 == 0) && (ldw % 8 == 0) && (((uintptr_t)A & 15) == 0) && (((uintptr_t)W & 15) == 0);
    if (c_dtype == IC_F32) dispatch_gemm<float>(A, W, C, M, N, K, lda, ldw, ldc, alpha, aligned, stream);
    else dispatch_gemm<bf16>(A, W, C, M, N, K, lda, ldw, ldc, alpha, aligned, stream);
    return ic_launch_status();
}
