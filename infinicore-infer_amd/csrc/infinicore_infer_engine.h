// C interface of the step function: one call issues every kernel of a step.
//
// The reference's step is inferBatch / forwardBatch (include/infinicore_infer/models/jiuge.h:89-110,
// src/models/jiuge/jiuge.cpp:114-298): a model object made from a meta struct and weight pointers, then
// one call per step with the tokens of all requests, their lengths, their start positions and their
// caches.  Here the model object (IcDecoder) is made from a description of the run order: which layer
// runs when, with which weights, on which cache planes.  A layer is a pre-norm residual block of softmax
// attention over the paged cache and a SwiGLU feed-forward; every size and constant is a field, none is
// compiled in.  The decoder owns no device memory: weights, cache planes, the step's integers and the
// workspace are the caller's, and a step allocates nothing.
//
// Two levels:
//   ic_decoder_forward  takes the step's integers where they already lie on the device (IcStepBatch) and
//                       launches the kernels; nothing else.  This is what a HIP graph records.
//   ic_decoder_step     takes them as host arrays in the shape of inferBatch (tokens, req_lens, req_pos, one
//                       block table per request and cache group, wanted places), lays them out in a pinned
//                       staging buffer of the caller, copies them to the device in one copy and calls
//                       ic_decoder_forward.
// Both return 0, or the status of the first kernel entry point that refused (see infinicore_infer_hip.h);
// ic_decoder_last_error then says which one.
#pragma once
#include "infinicore_infer_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

#define IC_MAX_CACHE_GROUPS 8

typedef struct IcDecoder IcDecoder;

// y = x * rsqrt(mean(x^2) + eps) * weight over the hidden size; weight float32.
typedef struct {
    const float* weight;
    float eps;
} IcNorm;

typedef struct {
    int n_heads, n_kv_heads, head_dim;
    int window;              // keys a query sees; 0: all
    int shared_kv;           // 1: reads the cache another entry wrote and projects queries only
    int rot_dim;             // rotary pairs (j, j + rot_dim/2) cover the first rot_dim elements of a head; 0: no rotation
    int max_positions;       // rows of cos and sin
    float softmax_scale;
    const float* cos;        // [max_positions, rot_dim / 2]
    const float* sin;
    const void* w_qkv;       // [(n_heads + 2 n_kv_heads) head_dim, hidden], rows [Q; K; V] (queries only when shared_kv)
    const void* w_o;         // [hidden, n_heads head_dim]
} IcAttention;

typedef struct {
    int intermediate;
    const void* w_gate_up;   // [2 intermediate, hidden], rows [gate; up]
    const void* w_down;      // [hidden, intermediate]
} IcSwiGLU;

// x += residual_scale * attention(mixer_norm(x)); x += residual_scale * swiglu(ffn_norm(x)).
typedef struct {
    IcNorm mixer_norm;
    IcAttention attention;
    IcNorm ffn_norm;
    IcSwiGLU ffn;
    float residual_scale;
} IcLayer;

// One entry of the run order.  A layer may appear in several entries (its weights are shared); an entry
// with writes_cache == 0 reads the planes another entry writes.
typedef struct {
    int layer;               // index into the layers
    int writes_cache;
    int group;               // cache group: which slots and block tables of a step this entry uses
    void* k_cache;           // [pages, n_kv_heads, page_size, head_dim] in the compute dtype
    void* v_cache;
} IcRunEntry;

// The model-level constants: what the reference's JiugeMeta holds (jiuge.h:12-18) plus the embedding and
// logit scales, which are applied at run time here, and the cache's geometry.
typedef struct {
    int dtype;               // compute dtype of weights, activations and cache: 0 float32, 1 bfloat16
    int hidden, vocab, page_size;
    int n_layers, n_entries, n_groups;
    int compute_units;       // of the device, for the key-split choice
    float embed_scale;       // x = table[token] * embed_scale
    float logit_scale;       // logits = (final_norm(x) * logit_scale) head^T
    const void* embed_table; // [vocab, hidden]
    const void* head_weight; // [vocab, hidden]
    IcNorm final_norm;
    const float* final_norm_scaled;   // final_norm.weight * logit_scale
    int* attention_counters;          // ic_attn_prefill_counter_ints() ints of the caller's, zero when the decoder is made; every step
                                      // leaves them zero.  Steps that overlap in time (two streams) need decoders with counters of their own
} IcDecoderMeta;

// A step's batch where it lies on the device.  Tokens of all requests are concatenated in request order.
typedef struct {
    int n_tokens, n_requests;
    int n_want;              // rows whose logits are wanted
    int n_decode_rows;       // rows that are a request's single new token
    int n_prefill_tiles;     // attention tiles of the prompt portions
    int want_rows_identity;  // every row is wanted, in order
    int decode_rows_identity;// every row is a single new token
    int max_position;        // largest position in the step
    int max_context;         // most keys a single-token row sees, rounded up as the caller's key-split buckets are
    int fixed_decode_splits; // > 0: use this key split
    const int* tokens;       // [n_tokens]
    const int* positions;    // [n_tokens]
    const int* token_req;    // [n_tokens] request row of each token
    const int* want_rows;    // [n_want]
    const int* decode_rows;  // [n_decode_rows] (unused when decode_rows_identity)
    const int* prefill_tiles;// [n_prefill_tiles, 4] = (request row, first token row, rows, first position)
    const int* group_slots[IC_MAX_CACHE_GROUPS];    // per group: [n_tokens] cache slot (page * page_size + offset) of each token
    const int* group_tables[IC_MAX_CACHE_GROUPS];   // per group: [n_requests, group_table_stride] logical page -> page id
    int group_table_stride[IC_MAX_CACHE_GROUPS];
} IcStepBatch;

// A step's batch as host arrays, in the shape of inferBatch (jiuge.h:89-110).
typedef struct {
    int n_tokens, n_requests;
    const int* tokens;       // [n_tokens]
    const int* req_lens;     // [n_requests] new tokens of each request
    const int* req_pos;      // [n_requests] position of each request's first new token
    const int* want_count;   // [n_requests] how many of a request's tokens want their logits
    const int* want;         // concatenated over requests: indices into a request's new tokens
    const int* const* tables;// [n_groups * n_requests]: block table of request r in group g at [g * n_requests + r]
    const int* table_len;    // [n_groups * n_requests] entries of each
    int tile_rows;           // rows per prefill attention tile (ic_attn_prefill_tile_rows())
    int fixed_decode_splits;
} IcHostBatch;

// Copies the descriptions (not the tensors they point to).  NULL when a field is out of range;
// ic_decoder_create_error() then says which.
IcDecoder* ic_decoder_create(const IcDecoderMeta* meta, const IcLayer* layers, const IcRunEntry* entries);
const char* ic_decoder_create_error();
void ic_decoder_destroy(IcDecoder* decoder);
const char* ic_decoder_last_error(const IcDecoder* decoder);

// Bytes of device workspace ic_decoder_forward needs for this batch (activations and partial results).
long long ic_decoder_workspace_bytes(const IcDecoder* decoder, const IcStepBatch* batch);
// Launches the step on `stream`.  logits: float32 [n_want, vocab], written when n_want > 0.  library_workspace: device
// memory for the library's matrix products (one per stream that runs steps at the same time).
int ic_decoder_forward(IcDecoder* decoder, const IcStepBatch* batch, void* workspace, long long workspace_bytes,
                       void* library_workspace, long long library_workspace_bytes, float* logits, hipStream_t stream);

// int32 elements of staging (host, pinned) and of device memory that ic_decoder_step needs for this batch.
long long ic_decoder_step_ints(const IcDecoder* decoder, const IcHostBatch* batch);
// Lays the batch out in `staging`, copies it to `device_ints` with one asynchronous copy, fills *laid_out (if not
// NULL) with the device view, and launches the step.  The caller must not touch `staging` until the copy has run.
int ic_decoder_step(IcDecoder* decoder, const IcHostBatch* batch, int* staging, int* device_ints, long long n_ints,
                    void* workspace, long long workspace_bytes, void* library_workspace, long long library_workspace_bytes,
                    float* logits, IcStepBatch* laid_out, hipStream_t stream);
// The same in two halves, for callers that size the workspace and the logits from the laid-out batch first:
// ic_decoder_pack only lays the batch out (no GPU call); the caller copies staging[0 .. n_ints) to device_ints.
int ic_decoder_pack(const IcDecoder* decoder, const IcHostBatch* batch, int* staging, const int* device_ints,
                    long long n_ints, IcStepBatch* laid_out);

// ---- which kernel takes what ------------------------------------------------------------------------------------------
// The rules by which a step's products and attention choose their kernels.  ic_decoder_forward asks them, and so
// does whoever issues the same kernels one by one (the parts' Python forward), so that both launch the same kernels
// for the same step and a rule is written once.  `dtype`: the compute dtype; lda, ldw: row strides in elements.
#define IC_TAIL_PLAIN 0       // the product, then the add+norm kernel
#define IC_TAIL_SPLIT_NORM 1  // the few-row product adds to the residual stream and hands on x * weight and sums of squares
#define IC_TAIL_SLICES 2      // slices over K, then the kernel that sums them, adds and applies the whole norm
#define IC_ATTN_GENERAL 0     // the general kernel for every row
#define IC_ATTN_SINGLE_TOKENS 1   // (bit) the split-key kernel for rows that are a request's single new token
#define IC_ATTN_PORTIONS 2        // (bit) the tiled matrix-core kernel for prompt portions
int ic_rule_few_rows();           // rows up to which the package's own product runs instead of the library's
int ic_rule_sumsq_parts_max();    // column blocks of sums of squares a product takes as row factors
// 1: a plain product of `rows` rows runs in the package's own kernel (ic_gemm_nt), 0: in the library (ic_matmul).
int ic_rule_own_product(int a_dtype, int w_dtype, int c_dtype, int rows);
// 1: the QKV projection runs with rotary and cache write in its epilogue (ic_gemm_qkv_rope); 0: product, then ic_rope_kv_write.
// kv_heads_written: 0 when the entry writes no cache; row_factors_owed: the rows' norm is half done (IcRowFactor).
int ic_rule_qkv_fused(int dtype, int rows, int K, int lda, int ldw, int head_dim, int rot_dim, int kv_heads_written, int row_factors_owed);
// 1: the gate/up projection runs with SwiGLU in its epilogue (ic_gemm_nt, c_mode 1); 0: product, then ic_swiglu.
int ic_rule_gate_up_fused(int dtype, int rows, int K, int lda, int ldw, int row_factors_owed);
// How a projection into the residual stream (O, down: N = hidden) that a norm follows runs: IC_TAIL_*.
int ic_rule_tail(int dtype, int rows, int N, int K, int lda, int ldw);
// Which attention kernels a step with n_decode_rows single-token rows and n_tiles prompt tiles takes: IC_ATTN_GENERAL, or bits.
int ic_rule_attention(int dtype, int head_dim, int page_size, int n_decode_rows, int n_tiles);
// Key counts are rounded up before the key split of single-token rows is chosen, so that a recorded step serves a range
// of lengths and splits as an eager one does: to a power of two up to 1,024 (at least 256), above that to a multiple of
// a quarter of the power of two below (2,560, 3,072, 3,584, 4,096, 5,120 ...).
int ic_rule_context_bucket(int n_keys);

// How many ways to split the keys of single-token rows (from sweeps on MI355X with caches that do not fit the
// last-level cache); see the decode attention kernel.  elem_bytes: of a cache element.  matrix_cores: 1 when the
// grouped-query kernel runs (bfloat16, several query heads per kv head).
int ic_attn_decode_splits(int n_decode_rows, int n_heads, int n_kv_heads, int head_dim, int elem_bytes, int window,
                          int max_context, int matrix_cores, int compute_units);

#ifdef __cplusplus
}
#endif
