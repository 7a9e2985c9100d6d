// C interface of the gfx950 kernel library (libinfinicore_infer_hip-<hash>.so).
//
// Every function launches on `stream` and returns 0 when the launch was queued,
// IC_ERR_ARG (-1) for a shape, stride, alignment or size the kernel does not take,
// IC_ERR_UNSUPPORTED (-2) for a dtype or head size without a kernel, IC_ERR_TOO_LARGE (-5)
// for a size beyond the fixed capacity of an entry point that allocates nothing, or the
// (positive) hipError_t of a failed launch.  Nothing here allocates device memory;
// scratch buffers are passed in by the caller.  dtype codes: 0 = float32, 1 = bfloat16.
//
// Cache layout of one layer: K and V planes [num_pages, n_kv_heads, page_size, head_dim].
// Block tables: int32 [requests, bt_stride], logical page -> page id.
#pragma once
#include <hip/hip_runtime.h>

#ifdef __cplusplus
extern "C" {
#endif

// ---- elementwise.hip ---------------------------------------------------------------------
// x[t, :] = table[tokens[t], :] * scale (x float32).
int ic_embed(const int* tokens, const void* table, int table_dtype, float* x, int T, int d, float scale, hipStream_t stream);
// out[r, :] = x[rows ? rows[r] : r, :] * rsqrt(mean(x^2) + eps) * w * out_scale (x, w float32).
int ic_rmsnorm(const float* x, const int* rows, const float* w, void* out, int out_dtype, int n_rows, int d, float eps, float out_scale, hipStream_t stream);
// x += alpha * y, then out = rmsnorm(x) * w.
int ic_add_rmsnorm(float* x, const void* y, int y_dtype, float alpha, const float* w, void* out, int out_dtype, int T, int d, float eps, hipStream_t stream);
// x += alpha * y over n elements.
int ic_residual_add(float* x, const void* y, int y_dtype, float alpha, long long n, hipStream_t stream);
// out[t, j] = up * silu(gate), gate = gate_up[t, j], up = gate_up[t, di + j].
int ic_swiglu(const void* gate_up, void* out, int dtype, int T, int di, hipStream_t stream);

// Whole cache pages copied inside a group's planes (n_planes planes of n_pages pages of page_bytes bytes, contiguous):
// planes[p][dst[i]] = planes[p][src[i]] for every plane p.  src, dst: device int32 [n_pairs]; no page both read and written.
int ic_copy_pages(void* planes, int n_planes, long long n_pages, long long page_bytes, const int* src, const int* dst, int n_pairs, hipStream_t stream);

// ---- rope_kv.hip ------------------------------------------------------------------------------
// Rotary on the q and k heads of qkv[T, row_stride] (pairs (j, j + rot/2)), k and v written to cache slot slots[t].
int ic_rope_kv_write(void* qkv, int dtype, const int* positions, const float* cos_t, const float* sin_t, void* kcache, void* vcache, const int* slots, int T, int row_stride, int nh, int nkvh, int dh, int rot, int page_size, hipStream_t stream);

// ---- attention ------------------------------------------------------------------------------------
// General kernel: any head size <= 512, float32 or bfloat16, optional window (0 = none).
int ic_attn_generic(const void* q, int q_stride, void* out, int out_stride, int dtype, const void* kcache, const void* vcache, const int* block_tables, int bt_stride, const int* token_req, const int* positions, int T, int nh, int nkvh, int dh, int page_size, float scale, int window, hipStream_t stream);
// Split-key kernel for single new tokens.  part_acc: float32 [n_tok, nh, nsplit, dh]; part_ml: float32 [n_tok, nh, nsplit, 2]; nsplit <= 64.
int ic_attn_decode_supported(int dtype, int dh);
// 1 when ic_attn_decode runs its grouped-query kernel on the matrix cores (bfloat16, several query heads per kv head): that
// kernel wants other key splits than the one-head-per-wave kernel (the matrix_cores argument of ic_attn_decode_splits).
int ic_attn_decode_on_matrix_cores(int dtype, int n_heads, int n_kv_heads);
int ic_attn_decode(const void* q, int q_stride, void* out, int out_stride, int dtype, const void* kcache, const void* vcache, const int* block_tables, int bt_stride, const int* tok_list, const int* token_req, const int* positions, float* part_acc, float* part_ml, int n_tok, int nh, int nkvh, int dh, int page_size, float scale, int window, int nsplit, hipStream_t stream);
// Matrix-core kernels for prompt portions (bfloat16; and true float32 with float32 matrix instructions, one wave group, walks never cut).
// tiles: int32 [n_tiles, 4] = (request row, first token row, rows <= tile_rows, first position).
int ic_attn_prefill_supported(int dtype, int dh, int page_size);
int ic_attn_prefill_tile_rows();
int ic_attn_prefill(const void* q, int q_stride, void* out, int out_stride, int dtype, const void* kcache, const void* vcache, const int* block_tables, int bt_stride, const int* tiles, int n_tiles, int nh, int nkvh, int dh, int page_size, float scale, int window, hipStream_t stream);
// The same with the number of wave groups per query tile given: 2 halves the longest tile's walk over the keys (few blocks), 1 keeps more blocks resident (many blocks), 0 chooses.
int ic_attn_prefill_groups(const void* q, int q_stride, void* out, int out_stride, int dtype, const void* kcache, const void* vcache, const int* block_tables, int bt_stride, const int* tiles, int n_tiles, int nh, int nkvh, int dh, int page_size, float scale, int window, int groups, hipStream_t stream);

// The same with a query tile's walk over the keys cut into parts that run as blocks of their own (one wave group): the grid holds
// `parts` blocks per (tile, head), a part walks at least part_len key tiles of 64, the block that arrives last merges the parts
// through `scratch` (ic_attn_prefill_scratch_floats floats).  ic_attn_prefill_parts proposes parts and part_len for a step whose
// longest tile sees max_keys keys (1: no cut).  The parts count themselves in at `counters`: ic_attn_prefill_counter_ints() ints of
// the caller's that are zero before the first launch; every launch leaves them zero, so one buffer serves all launches that follow
// each other on a stream.  Launches that overlap in time (two streams) need counters of their own.
long long ic_attn_prefill_scratch_floats(int n_tiles, int nh, int dh, int parts);
int ic_attn_prefill_counter_ints();
int ic_attn_prefill_parts(int n_tiles, int nh, int dh, int max_keys, int compute_units, int* part_len);
int ic_attn_prefill_parts_of_step(int dtype, int n_tiles, int nh, int dh, int max_position, int window, int compute_units, int* part_len);   // max_keys from the step's largest position and the window
int ic_attn_prefill_split(const void* q, int q_stride, void* out, int out_stride, int dtype, const void* kcache, const void* vcache, const int* block_tables, int bt_stride, const int* tiles, int n_tiles, int nh, int nkvh, int dh, int page_size, float scale, int window, int groups, int parts, int part_len, float* scratch, long long scratch_floats, int* counters, hipStream_t stream);

// ---- gemm.hip ---------------------------------------------------------------------------------------
// A norm y = x * rsqrt(mean(x^2) + eps) * w between two products of M <= 16 rows can be split over them: the
// product before it adds its result to the residual stream, stores x * w and the sums of x^2 per row and
// column block (IcResidualNorm); the product after it multiplies each row of its result by the row's
// rsqrt(sum / width + eps) (IcRowFactor).
typedef struct {
    const float* sumsq;   // [n_parts, 16]: sum of squares of row m over column block b at [b * 16 + m]
    int n_parts;          // <= 256
    int width;            // elements per row the sums run over
    float eps;
} IcRowFactor;
typedef struct {
    float* x;             // float32 residual stream [M, N], updated in place
    int ldx;
    const float* weight;  // [N] the following norm's weight
    float alpha;          // x += alpha * result
    float* sumsq_out;     // [n_parts, 16]
    int n_parts;          // must equal ic_gemm_nt_residual_parts(N)
} IcResidualNorm;
// C[M, N] = alpha * A[M, K] W[N, K]^T, bfloat16 operands, float32 accumulation.  c_mode 1 (M <= 16):
// W = [gate; up], C[M, N/2] = up * silu(gate).  c_mode 2 (M <= 16, bfloat16 C, tail != NULL):
// x += tail->alpha * (alpha A W^T), C = x * tail->weight.  row_factor (nullable, M <= 16): see above.
int ic_gemm_nt_supported(int a_dtype, int w_dtype, int c_dtype);
int ic_gemm_nt_residual_parts(int N);
int ic_gemm_nt(const void* A, int a_dtype, const void* W, int w_dtype, void* C, int c_dtype, int M, int N, int K, int lda, int ldw, int ldc, float alpha, int c_mode, const IcRowFactor* row_factor, const IcResidualNorm* tail, hipStream_t stream);
// Rows that the products with an epilogue take: kind 1 (c_mode 1, SwiGLU) and kind 2 (ic_gemm_qkv_rope) 32 where the weights can be
// read in whole cache lines (K a multiple of 64, row strides multiples of 8), 16 otherwise; without row factors above 16 rows.
int ic_gemm_nt_epilogue_rows(int kind, int K, int lda, int ldw);
// QKV projection of M <= 16 rows with rotary and cache write in the epilogue; row_factor nullable.
int ic_gemm_qkv_rope_supported(int dtype, int dh);
int ic_gemm_qkv_rope(const void* A, const void* W, void* C, int M, int K, int lda, int ldw, int ldc, const int* positions, const int* slots, const float* cos_t, const float* sin_t, void* kcache, void* vcache, int nh, int nkvh, int dh, int page_size, const IcRowFactor* row_factor, hipStream_t stream);

// ---- gemm_splitk.hip ----------------------------------------------------------------------------------
// Products of 1..64 rows (bfloat16) as float32 slices over K, P[s, m, n] = A[m, K_s] . W[n, K_s], and the kernel
// that sums the slices, adds them to the residual stream and applies the norm that follows.  For the O and down
// projections of 17..64 rows, where it beats the library's product (ic_gemm_splitk_pays says when).
int ic_gemm_splitk_supported(int M, int N, int K, int lda, int ldw);
int ic_gemm_splitk_slices(int N, int K);      // how many slices to use (never an empty one)
int ic_gemm_splitk_pays(int M, int N, int K);
int ic_gemm_splitk(const void* A, const void* W, float* P, int M, int N, int K, int lda, int ldw, int n_slices, hipStream_t stream);
// P [S, M, d]: x += alpha * (the product, rounded to bfloat16); out = rmsnorm(x) * w.
int ic_splitk_add_rmsnorm(const float* P, int n_slices, int M, float* x, float alpha, const float* w, void* out, int d, float eps, hipStream_t stream);

// ---- matmul_library.hip ------------------------------------------------------------------------------
// The library (hipBLASLt) matrix product for many rows: C[M, N] = alpha * A[M, K] W[N, K]^T, bfloat16 operands with a
// bfloat16 or float32 result, or all float32 (true float32).  Descriptors and the algorithm are kept per shape.
// Returns -3 when the library refuses a call and -4 when it proposes no algorithm.  These two allocate host-side
// descriptors at the first call of a shape; workspace is device memory passed in by the caller.
int ic_matmul_supported(int a_dtype, int c_dtype);
int ic_matmul(const void* A, int a_dtype, const void* W, void* C, int c_dtype, int M, int N, int K, int lda, int ldw, int ldc, float alpha, void* workspace, long long workspace_bytes, hipStream_t stream);
// Times the algorithms the library has for this shape and keeps the fastest; returns how many were tried.
// flush (or nullptr): memory larger than the caches, overwritten before every timed launch so that operands come from memory.
int ic_matmul_tune(const void* A, int a_dtype, const void* W, void* C, int c_dtype, int M, int N, int K, int lda, int ldw, int ldc, void* workspace, long long workspace_bytes, void* flush, long long flush_bytes, int reps, hipStream_t stream);

// ---- sampling.hip -----------------------------------------------------------------------------------
// Greedy choice per row; scratch_val / scratch_idx: 64 * n_rows elements.
int ic_argmax(const float* logits, long long row_stride, int n_rows, int V, float* scratch_val, int* scratch_idx, int* out, hipStream_t stream);
// For callers that cannot allocate device memory (code under HIP graph capture, tight serving loops,
// harnesses that forbid it); it has no counterpart in the reference.  The same result as ic_argmax, with the
// partial results in the library's own static device memory (512 KB on every GPU the library runs on, held
// until the process ends) instead of a scratch buffer from the caller: nothing is allocated or freed, here
// or in anything it calls.  At most ic_argmax_static_max_rows() (1024) rows: more returns IC_ERR_TOO_LARGE
// (-5) and launches nothing.  The device of `stream` must be the current device.  All calls on one GPU share
// that memory: calls that overlap on one GPU (two streams, two threads) race; calls in stream order do not.
int ic_argmax_static_max_rows();
int ic_argmax_static(const float* logits, long long row_stride, int n_rows, int V, int* out, hipStream_t stream);
// Temperature / top-k / top-p with one uniform draw per row; temperature == nullptr: argmax.
int ic_sample(const float* logits, long long row_stride, int n_rows, int V, const float* temperature, const int* top_k, const float* top_p, const float* uniform, int* out, hipStream_t stream);

// ---- what the device reaches at most (measurements for the reports, not on the model's path) ------------------------
// Issues only MFMA instructions (bfloat16, 32x32x16) on blocks_per_unit blocks of four waves per compute unit; returns
// the floating-point operations issued (the caller times the launch), or a negative status.
long long ic_peak_mfma_bf16(float* sink, int iters, int blocks_per_unit, hipStream_t stream);
// Reads `bytes` of device memory once with 16-byte loads and does nothing else.
int ic_peak_read(const void* src, long long bytes, int blocks_per_unit, unsigned* sink, hipStream_t stream);

#ifdef __cplusplus
}
#endif
