// C[M, N] = alpha * A[M, K] * W[N, K]^T for few rows M (decoding, the output
// head): bfloat16 operands on the matrix cores, float32 accumulation, float32
// or bfloat16 result.  The weight matrix is streamed once per 64 rows of A.
//
// Grid (ceil(N/(16*NT)), ceil(M/(16*MT))), WPB waves.  Every wave owns the same
// NT tiles of 16 weight rows and a share of K (k-steps of 32, dealt in turn; WPB is 4, 8
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

template <typename TC, int NT, int MT, int WPB, int UNROLL, bool ALIGNED, bool CSWIGLU>
__global__ void __launch_bounds__(WPB * 64)
gemm_nt_bf16_kernel(const uint16_t* __restrict__ A, const uint16_t* __restrict__ W, TC* __restrict__ C,
                    int M, int N, int K, int lda, int ldw, int ldc, float alpha) {
    __shared__ float red[WPB - 1][NT * MT][64][4];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r = lane & 15, kq = lane >> 4;
    // CSWIGLU: W = [gate rows (N/2); up rows (N/2)]; a block owns 16 gate rows and the matching
    // 16 up rows and writes C[m][n] = up * silu(gate) for its 16 columns of the N/2 wide output.
    const int NO = CSWIGLU ? N / 2 : N;                      // output columns
    const int n0 = blockIdx.x * (CSWIGLU ? 16 : 16 * NT), m0 = blockIdx.y * (16 * MT);

    const uint16_t* wp[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        const int base = CSWIGLU ? n0 + nt * NO : n0 + 16 * nt;
        const int lim = CSWIGLU ? (nt + 1) * NO : N;
        const int nrow = (base + r < lim) ? base + r : lim - 1;
        wp[nt] = W + (size_t)nrow * ldw + 8 * kq;
    }
    const uint16_t* ap[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const int mrow = (m0 + 16 * mt + r < M) ? m0 + 16 * mt + r : M - 1;
        ap[mt] = A + (size_t)mrow * lda + 8 * kq;
    }
    v4f acc[NT][MT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[nt][mt] = v4f{0.f, 0.f, 0.f, 0.f};

    // k-steps of 32 are dealt to the waves in turn; UNROLL steps are loaded before any is used
    const int nsteps = (K + 31) >> 5;
    for (int s0 = wave; s0 < nsteps; s0 += WPB * UNROLL) {
        v4s wlo[UNROLL][NT], whi[UNROLL][NT], alo[UNROLL][MT], ahi[UNROLL][MT];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            const int kk = 32 * (s0 + u * WPB);
            const int valid = K - kk - 8 * kq;          // <= 0 beyond the end of K
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                if (valid > 0) load8<ALIGNED>(wp[nt] + kk, valid, wlo[u][nt], whi[u][nt]);
                else { wlo[u][nt] = v4s{0, 0, 0, 0}; whi[u][nt] = wlo[u][nt]; }
            }
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
            for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) {
                    acc[nt][mt] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(wlo[u][nt], alo[u][mt], acc[nt][mt], 0, 0, 0);
                    acc[nt][mt] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(whi[u][nt], ahi[u][mt], acc[nt][mt], 0, 0, 0);
                }
    }
    if (wave > 0) {
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                for (int e = 0; e < 4; ++e) red[wave - 1][nt * MT + mt][lane][e] = acc[nt][mt][e];
    }
    __syncthreads();
    if (wave > 0) return;
    if (CSWIGLU) {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const int m = m0 + 16 * mt + r;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                float g = acc[0][mt][e], u = acc[NT - 1][mt][e];
#pragma unroll
                for (int w = 0; w < WPB - 1; ++w) { g += red[w][mt][lane][e]; u += red[w][(NT - 1) * MT + mt][lane][e]; }
                // both projections are rounded to the output type first, as when they are stored
                g = to_f32(from_f32<TC>(alpha * g));
                u = to_f32(from_f32<TC>(alpha * u));
                const int n = n0 + 4 * kq + e;
                if (m < M && n < NO) C[(size_t)m * ldc + n] = from_f32<TC>(u * (g / (1.0f + expf(-g))));
            }
        }
        return;
    }
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const int m = m0 + 16 * mt + r;             // column j of D = l % 16
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                float v = acc[nt][mt][e];
#pragma unroll
                for (int w = 0; w < WPB - 1; ++w) v += red[w][nt * MT + mt][lane][e];
                const int n = n0 + 16 * nt + 4 * kq + e;    // row i of D
                if (m < M && n < N) C[(size_t)m * ldc + n] = from_f32<TC>(alpha * v);
            }
        }
}

template <typename TC, int NT, int MT, int WPB, int UNROLL>
static void launch_gemm(const void* A, const void* W, void* C, int M, int N, int K, int lda, int ldw,
                        int ldc, float alpha, bool aligned, hipStream_t stream) {
    dim3 grid((N + 16 * NT - 1) / (16 * NT), (M + 16 * MT - 1) / (16 * MT)), block(WPB * 64);
    if (aligned)
        hipLaunchKernelGGL((gemm_nt_bf16_kernel<TC, NT, MT, WPB, UNROLL, true, false>), grid, block, 0, stream,
                           (const uint16_t*)A, (const uint16_t*)W, (TC*)C, M, N, K, lda, ldw, ldc, alpha);
    else
        hipLaunchKernelGGL((gemm_nt_bf16_kernel<TC, NT, MT, WPB, UNROLL, false, false>), grid, block, 0, stream,
                           (const uint16_t*)A, (const uint16_t*)W, (TC*)C, M, N, K, lda, ldw, ldc, alpha);
}

// The gate/up projection with the activation in its epilogue: W [N, K] = [gate; up], C [M, N/2].
template <typename TC, int WPB, int UN = 2>
static void launch_gemm_swiglu(const void* A, const void* W, void* C, int M, int N, int K, int lda, int ldw,
                               int ldc, bool aligned, hipStream_t stream) {
    dim3 grid((N / 2 + 15) / 16, (M + 15) / 16), block(WPB * 64);
    if (aligned)
        hipLaunchKernelGGL((gemm_nt_bf16_kernel<TC, 2, 1, WPB, UN, true, true>), grid, block, 0, stream,
                           (const uint16_t*)A, (const uint16_t*)W, (TC*)C, M, N, K, lda, ldw, ldc, 1.0f);
    else
        hipLaunchKernelGGL((gemm_nt_bf16_kernel<TC, 2, 1, WPB, UN, false, true>), grid, block, 0, stream,
                           (const uint16_t*)A, (const uint16_t*)W, (TC*)C, M, N, K, lda, ldw, ldc, 1.0f);
}

// NT weight tiles of 16 rows share one load of the A fragments; WPB waves split K.  Both are
// chosen so that (column blocks x waves) fills the chip's SIMDs about twice over.
template <typename TC>
static void dispatch_gemm(const void* A, const void* W, void* C, int M, int N, int K, int lda, int ldw,
                          int ldc, float alpha, bool aligned, hipStream_t stream) {
    const int tiles = (N + 15) / 16;
#define IC_GO(NT, MT, WPB, UN) launch_gemm<TC, NT, MT, WPB, UN>(A, W, C, M, N, K, lda, ldw, ldc, alpha, aligned, stream)
    // tilings from a sweep over the projection shapes of 1B..8B models on MI355X
    if (M <= 16) {
        if (tiles < 256) IC_GO(1, 1, 16, 2);
        else if (tiles < 600) IC_GO(2, 1, 16, 4);
        else if (tiles < 2048) { if (M <= 4) IC_GO(1, 1, 8, 2); else IC_GO(1, 1, 4, 2); }
        else { if (M <= 8) IC_GO(1, 1, 16, 2); else IC_GO(4, 1, 4, 2); }
    } else if (M <= 32) {
        if (tiles < 600) IC_GO(1, 2, 8, 2);
        else IC_GO(2, 2, 4, 2);
    } else {
        if (tiles < 256) IC_GO(1, 4, 8, 1);
        else IC_GO(2, 4, 4, 1);
    }
#undef IC_GO
}

// The same product with the tiling chosen by the caller (for tuning and tests):
// nt in {1, 2, 4}, wpb in {4, 8, 16}, unroll in {2, 4}; mt follows from M.
template <typename TC, int NT, int WPB, int UN>
static int launch_cfg_m(const void* A, const void* W, void* C, int M, int N, int K, int lda, int ldw, int ldc,
                        float alpha, bool aligned, hipStream_t stream) {
    if (M <= 16) launch_gemm<TC, NT, 1, WPB, UN>(A, W, C, M, N, K, lda, ldw, ldc, alpha, aligned, stream);
    else if (M <= 32) launch_gemm<TC, NT, 2, WPB, (UN > 2 ? 2 : UN)>(A, W, C, M, N, K, lda, ldw, ldc, alpha, aligned, stream);
    else {
        if (NT * WPB > 32) return IC_ERR_UNSUPPORTED;       // would not fit LDS
        launch_gemm<TC, (NT > 2 ? 2 : NT), 4, (WPB > 8 ? 8 : WPB), 1>(A, W, C, M, N, K, lda, ldw, ldc, alpha, aligned, stream);
    }
    return IC_OK;
}

IC_EXPORT int ic_gemm_nt_cfg(const void* A, const void* W, void* C, int c_dtype, int M, int N, int K, int lda,
                             int ldw, int ldc, float alpha, int nt, int wpb, int unroll, hipStream_t stream) {
    if (M <= 0 || N <= 0) return IC_OK;
    if (K <= 0 || lda < K || ldw < K || c_dtype != IC_BF16) return IC_ERR_ARG;
    const bool aligned = (lda % 8 == 0) && (ldw % 8 == 0) && (((uintptr_t)A & 15) == 0) && (((uintptr_t)W & 15) == 0);
    if (nt == 0) {                                  // nt == 0: the variant with SwiGLU in the epilogue
        if (M > 16 || (N & 1) || ldc < N / 2) return IC_ERR_ARG;
#define IC_SW(WPB, UN) if (wpb == WPB && unroll == UN) { launch_gemm_swiglu<bf16, WPB, UN>(A, W, C, M, N, K, lda, ldw, ldc, aligned, stream); return ic_launch_status(); }
        IC_SW(4, 2) IC_SW(4, 4) IC_SW(8, 2) IC_SW(8, 4) IC_SW(16, 2) IC_SW(16, 4)
#undef IC_SW
        return IC_ERR_UNSUPPORTED;
    }
    if (ldc < N) return IC_ERR_ARG;
    int st = IC_ERR_UNSUPPORTED;
#define IC_CFG(NT, WPB, UN) \
    if (nt == NT && wpb == WPB && unroll == UN) st = launch_cfg_m<bf16, NT, WPB, UN>(A, W, C, M, N, K, lda, ldw, ldc, alpha, aligned, stream);
    IC_CFG(1, 4, 2) IC_CFG(1, 4, 4) IC_CFG(1, 8, 2) IC_CFG(1, 8, 4) IC_CFG(1, 16, 2) IC_CFG(1, 16, 4)
    IC_CFG(2, 4, 2) IC_CFG(2, 4, 4) IC_CFG(2, 8, 2) IC_CFG(2, 8, 4) IC_CFG(2, 16, 2) IC_CFG(2, 16, 4)
    IC_CFG(4, 4, 2) IC_CFG(4, 8, 2)
#undef IC_CFG
    if (st) return st;
    return ic_launch_status();
}

IC_EXPORT int ic_gemm_nt_supported(int a_dtype, int w_dtype, int c_dtype) {
    return a_dtype == IC_BF16 && w_dtype == IC_BF16 && (c_dtype == IC_F32 || c_dtype == IC_BF16);
}

// c_mode 0: C [M, N] = alpha * A W^T.  c_mode 1 (M <= 16, N even, alpha ignored): W = [gate; up] and
// C [M, N/2] = up * silu(gate), both projections rounded to C's type before the activation.
IC_EXPORT int ic_gemm_nt(const void* A, int a_dtype, const void* W, int w_dtype, void* C, int c_dtype,
                         int M, int N, int K, int lda, int ldw, int ldc, float alpha, int c_mode,
                         hipStream_t stream) {
    if (M <= 0 || N <= 0) return IC_OK;
    if (K <= 0 || lda < K || ldw < K || c_mode < 0 || c_mode > 1) return IC_ERR_ARG;
    if (c_mode == 1 ? (M > 16 || (N & 1) || ldc < N / 2) : (ldc < N)) return IC_ERR_ARG;
    if (!ic_gemm_nt_supported(a_dtype, w_dtype, c_dtype)) return IC_ERR_UNSUPPORTED;
    if ((M + 63) / 64 > 65535) return IC_ERR_ARG;
    const bool aligned = (lda % 8 == 0) && (ldw % 8 == 0) && (((uintptr_t)A & 15) == 0) && (((uintptr_t)W & 15) == 0);
    if (c_mode == 1) {
        const int tiles = (N / 2 + 15) / 16;
        if (c_dtype == IC_F32) {
            if (tiles < 300) launch_gemm_swiglu<float, 8>(A, W, C, M, N, K, lda, ldw, ldc, aligned, stream);
            else launch_gemm_swiglu<float, 4>(A, W, C, M, N, K, lda, ldw, ldc, aligned, stream);
        } else {
            if (tiles < 300) launch_gemm_swiglu<bf16, 8>(A, W, C, M, N, K, lda, ldw, ldc, aligned, stream);
            else launch_gemm_swiglu<bf16, 4>(A, W, C, M, N, K, lda, ldw, ldc, aligned, stream);
        }
        return ic_launch_status();
    }
    if (c_dtype == IC_F32) dispatch_gemm<float>(A, W, C, M, N, K, lda, ldw, ldc, alpha, aligned, stream);
    else dispatch_gemm<bf16>(A, W, C, M, N, K, lda, ldw, ldc, alpha, aligned, stream);
    return ic_launch_status();
}
