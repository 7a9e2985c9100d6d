// Entry points for tests and sweeps: the few-row products with a variant of their kernels named by the caller.
// Not part of the interface a caller of the library needs: ic_gemm_nt and ic_gemm_qkv_rope choose for themselves.
// A variant holds for the one call that names it and changes nothing for any other call, thread or engine.
#pragma once
#include "infinicore_infer_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

// ic_gemm_nt with whole_lines == 0: the weights are loaded in operand layout also where whole cache lines through LDS would apply
// (K a multiple of 64, aligned operands); products of 17..32 rows with an epilogue, which exist with whole lines only, are refused.
int ic_gemm_nt_variant(const void* A, int a_dtype, const void* W, int w_dtype, void* C, int c_dtype, int M, int N, int K, int lda, int ldw, int ldc, float alpha, int c_mode, const IcRowFactor* row_factor, const IcResidualNorm* tail, int whole_lines, hipStream_t stream);
// ic_gemm_qkv_rope with the used weight rows per tile given: 16, 8 or 4 (0: chosen from the number of heads, as ic_gemm_qkv_rope does).
int ic_gemm_qkv_rope_variant(const void* A, const void* W, void* C, int M, int K, int lda, int ldw, int ldc, const int* positions, const int* slots, const float* cos_t, const float* sin_t, void* kcache, void* vcache, int nh, int nkvh, int dh, int page_size, const IcRowFactor* row_factor, int tile_rows, hipStream_t stream);
// The few-row product with the tiling chosen by the caller; nt == 0 selects the SwiGLU variant.
int ic_gemm_nt_cfg(const void* A, const void* W, void* C, int c_dtype, int M, int N, int K, int lda, int ldw, int ldc, float alpha, int nt, int wpb, int unroll, hipStream_t stream);

#ifdef __cplusplus
}
#endif
