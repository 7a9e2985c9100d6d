// The step function in native code: every kernel of a step issued by one call (host code only; the
// kernels are the library's own entry points).  The reference's is src/models/jiuge/jiuge.cpp:114-298.
//
// What runs for a layer depends on the step alone, never on the model: up to 16 rows in bfloat16 take the
// few-row products with their epilogues (rotary and cache write after QKV; residual add, the next norm's
// weight and sums of squares after O and down; SwiGLU after gate/up), the norm between two products being
// split over them; more rows, or float32, take the library's products and the norm, rotary and activation
// kernels.  Single-token rows go to the split-key attention kernel, prompt portions to the tiled one, what
// neither takes to the general one.
#include "common.h"
#include "infinicore_infer_engine.h"
#include <algorithm>
#include <cstdio>
#include <cstring>
#include <string>
#include <vector>

namespace {

// The thresholds below are read by the ic_rule_* functions alone; the step function here and the parts' Python
// forward both ask those functions, so a rule is written once.
constexpr int kFewRows = 16;        // up to here the few-row products beat the library
constexpr int kMidRows = 64;        // up to here the sliced product beats it for results as wide as the model
constexpr int kMaxSumsqParts = 256; // column blocks of sums of squares a product takes as row factors

thread_local std::string g_create_error;

inline size_t align_up(size_t n, size_t a) { return (n + a - 1) / a * a; }
inline int dtype_size(int dtype) { return dtype == IC_BF16 ? 2 : 4; }

struct Workspace {
    // byte offsets into the caller's workspace
    size_t residual, normed, qkv, attn_out, mixer_out, ffn_out, mixer_tail, mixer_sumsq, ffn_tail, ffn_sumsq, gate_up, act,
        part_acc, part_ml, head_in, tail_parts, tile_parts, total;
};

// Rows whose norm is half done: values = x * w, sums of squares per column block; the row factor
// rsqrt(sum / width + eps) is applied by the product that consumes them.
struct Deferred {
    const void* values = nullptr;
    const float* sumsq = nullptr;
    int parts = 0, width = 0;
    float eps = 0.f;
};

}  // namespace

// ---- which kernel takes what: the one home of the dispatch rules ----------------------------------------------------------
IC_EXPORT int ic_rule_few_rows() { return kFewRows; }
IC_EXPORT int ic_rule_sumsq_parts_max() { return kMaxSumsqParts; }

IC_EXPORT int ic_rule_own_product(int a_dtype, int w_dtype, int c_dtype, int rows) {
    return rows <= kFewRows && a_dtype == IC_BF16 && ic_gemm_nt_supported(a_dtype, w_dtype, c_dtype);
}

IC_EXPORT int ic_rule_qkv_fused(int dtype, int rows, int K, int lda, int ldw, int head_dim, int rot_dim, int kv_heads_written,
                                int row_factors_owed) {
    if (dtype != IC_BF16 || kv_heads_written <= 0 || rot_dim != head_dim || !ic_gemm_qkv_rope_supported(IC_BF16, head_dim)) return 0;
    if (rows <= kFewRows) return 1;
    return !row_factors_owed && rows <= ic_gemm_nt_epilogue_rows(2, K, lda, ldw);
}

IC_EXPORT int ic_rule_gate_up_fused(int dtype, int rows, int K, int lda, int ldw, int row_factors_owed) {
    if (dtype != IC_BF16) return 0;
    if (rows <= kFewRows) return 1;
    return !row_factors_owed && rows <= ic_gemm_nt_epilogue_rows(1, K, lda, ldw);
}

IC_EXPORT int ic_rule_tail(int dtype, int rows, int N, int K, int lda, int ldw) {
    if (dtype != IC_BF16 || rows <= 0) return IC_TAIL_PLAIN;
    if (rows <= kMidRows && N % 4 == 0 && ic_gemm_splitk_supported(rows, N, K, lda, ldw) && ic_gemm_splitk_pays(rows, N, K))
        return IC_TAIL_SLICES;
    if (rows <= kFewRows && ic_gemm_nt_residual_parts(N) <= kMaxSumsqParts) return IC_TAIL_SPLIT_NORM;
    return IC_TAIL_PLAIN;
}

IC_EXPORT int ic_rule_attention(int dtype, int head_dim, int page_size, int n_decode_rows, int n_tiles) {
    const bool dec_ok = ic_attn_decode_supported(dtype, head_dim) != 0;
    const bool pre_ok = ic_attn_prefill_supported(dtype, head_dim, page_size) != 0;
    const bool use_dec = dec_ok && n_decode_rows > 0 && (pre_ok || n_tiles == 0);
    const bool use_pre = pre_ok && n_tiles > 0 && (dec_ok || n_decode_rows == 0);
    if (!((use_dec || n_decode_rows == 0) && (use_pre || n_tiles == 0))) return IC_ATTN_GENERAL;
    return (use_dec ? IC_ATTN_SINGLE_TOKENS : 0) | (use_pre ? IC_ATTN_PORTIONS : 0);
}

IC_EXPORT int ic_rule_context_bucket(int n_keys) {
    int b = 256;
    while (b < n_keys) b *= 2;
    if (b <= 1024) return b;
    const int q = b / 8;
    return (n_keys + q - 1) / q * q;
}

struct IcDecoder {
    IcDecoderMeta meta;
    std::vector<IcLayer> layers;
    std::vector<IcRunEntry> entries;
    int max_qkv_width = 0, max_attn_width = 0, max_intermediate = 0;
    std::string error;

    int fail(int status, const char* what, int entry) {
        char buf[256];
        if (entry >= 0) snprintf(buf, sizeof buf, "run-order entry %d (layer %d): %s returned %d", entry, entries[entry].layer, what, status);
        else snprintf(buf, sizeof buf, "%s returned %d", what, status);
        error = buf;
        return status;
    }

    // the last question put to ic_attn_decode_splits and its answer: the layers of a model mostly ask the same one
    mutable int split_key[7] = {-1, -1, -1, -1, -1, -1, -1}, split_answer = 1;

    int splits_for(const IcStepBatch& b, const IcAttention& a) const {
        if (b.fixed_decode_splits > 0) return b.fixed_decode_splits;
        const int matrix_cores = ic_attn_decode_on_matrix_cores(meta.dtype, a.n_heads, a.n_kv_heads);
        const int key[7] = {b.n_decode_rows, a.n_heads, a.n_kv_heads, a.head_dim, a.window, b.max_context, matrix_cores};
        if (memcmp(key, split_key, sizeof key) != 0) {
            split_answer = ic_attn_decode_splits(b.n_decode_rows, a.n_heads, a.n_kv_heads, a.head_dim, dtype_size(meta.dtype), a.window,
                                                 b.max_context, matrix_cores, meta.compute_units);
            memcpy(split_key, key, sizeof key);
        }
        return split_answer;
    }

    // into how many parts the walks of a step's prompt tiles are cut (1: not at all), and key tiles per part
    int tile_parts_for(const IcStepBatch& b, const IcAttention& a, int* part_len) const {
        if (!meta.attention_counters) { if (part_len) *part_len = 0; return 1; }     // no counters: no cut
        return ic_attn_prefill_parts_of_step(meta.dtype, b.n_prefill_tiles, a.n_heads, a.head_dim, b.max_position, a.window, meta.compute_units, part_len);
    }

    Workspace layout(const IcStepBatch& b) const {
        const size_t T = (size_t)b.n_tokens, d = (size_t)meta.hidden, ds = (size_t)dtype_size(meta.dtype);
        const int parts = ic_gemm_nt_residual_parts(meta.hidden);
        Workspace w{};
        size_t o = 0;
        auto take = [&](size_t bytes) { const size_t at = o; o = align_up(o + bytes, 256); return at; };
        w.residual = take(T * d * 4);
        w.normed = take(T * d * ds);
        w.qkv = take(T * (size_t)max_qkv_width * ds);
        w.attn_out = take(T * (size_t)max_attn_width * ds);
        w.mixer_out = take(T * d * ds);
        w.ffn_out = take(T * d * ds);
        const size_t few = std::min<size_t>(T, (size_t)ic_rule_few_rows());
        w.mixer_tail = take(few * d * 2);
        w.mixer_sumsq = take((size_t)parts * 16 * 4);
        w.ffn_tail = take(few * d * 2);
        w.ffn_sumsq = take((size_t)parts * 16 * 4);
        w.gate_up = take(T * 2 * (size_t)max_intermediate * ds);
        w.act = take(T * (size_t)max_intermediate * ds);
        size_t acc = 0, ml = 0;      // partial results of the key splits: [row, head, split, head size] and [row, head, split, 2]
        if (b.n_decode_rows > 0)
            for (const IcLayer& l : layers) {
                const size_t cells = (size_t)b.n_decode_rows * l.attention.n_heads * (size_t)splits_for(b, l.attention);
                acc = std::max(acc, cells * l.attention.head_dim);
                ml = std::max(ml, cells * 2);
            }
        w.part_acc = take(acc * 4);
        w.part_ml = take(ml * 4);
        w.head_in = take((size_t)b.n_want * d * ds);
        size_t slices = 0;           // the O and down products as slices over K, where that pays
        for (const IcLayer& l : layers)
            for (const int K : {l.attention.n_heads * l.attention.head_dim, l.ffn.intermediate})
                if (ic_rule_tail(meta.dtype, (int)T, meta.hidden, K, K, K) == IC_TAIL_SLICES)
                    slices = std::max(slices, (size_t)ic_gemm_splitk_slices(meta.hidden, K));
        w.tail_parts = take(slices * T * d * 4);
        size_t cut = 0;              // the states of prompt tiles whose walk over the keys is cut into parts
        if (meta.dtype == IC_BF16 && b.n_prefill_tiles > 0)
            for (const IcLayer& l : layers) {
                int len = 0;
                const int p = tile_parts_for(b, l.attention, &len);
                cut = std::max(cut, (size_t)ic_attn_prefill_scratch_floats(b.n_prefill_tiles, l.attention.n_heads, l.attention.head_dim, p));
            }
        w.tile_parts = take(cut * 4);
        w.total = o;
        return w;
    }
    // out[M, N] = alpha * a w^T: the few-row product, or the library's.
    int linear(const void* a, int lda, const void* w, void* out, int out_dtype, int M, int N, int K, float alpha,
               const Deferred* rows, void* lib_ws, long long lib_ws_bytes, hipStream_t stream) const {
        if (ic_rule_own_product(meta.dtype, meta.dtype, out_dtype, M)) {
            IcRowFactor rf{};
            if (rows) rf = IcRowFactor{rows->sumsq, rows->parts, rows->width, rows->eps};
            return ic_gemm_nt(a, IC_BF16, w, IC_BF16, out, out_dtype, M, N, K, lda, K, N, alpha, 0, rows ? &rf : nullptr,
                              nullptr, stream);
        }
        if (rows) return IC_ERR_ARG;      // half-normed rows exist only where the few-row product runs
        return ic_matmul(a, meta.dtype, w, out, out_dtype, M, N, K, lda, K, N, alpha, lib_ws, lib_ws_bytes, stream);
    }

    // 17..64 rows (and 13..16 long ones) into the residual stream: x += alpha * (a w^T), out = rmsnorm(x) * weight, through the sliced
    // product and the kernel that sums the slices.
    int tail_in_slices(const void* a, int K, const void* w, float* parts, float* x, float alpha, const float* weight, float eps,
                       void* out, int T, hipStream_t stream) const {
        const int d = meta.hidden;
        const int slices = ic_gemm_splitk_slices(d, K);
        const int st = ic_gemm_splitk(a, w, parts, T, d, K, K, K, slices, stream);
        if (st) return st;
        return ic_splitk_add_rmsnorm(parts, slices, T, x, alpha, weight, out, d, eps, stream);
    }

    int forward(const IcStepBatch& b, void* workspace, long long workspace_bytes, void* lib_ws, long long lib_ws_bytes,
                float* logits, hipStream_t stream) {
        error.clear();
        const int T = b.n_tokens, d = meta.hidden, dt = meta.dtype, ps = meta.page_size;
        if (T <= 0) return IC_OK;
        if (b.n_requests <= 0 || b.n_want < 0 || b.n_decode_rows < 0 || b.n_prefill_tiles < 0 || !b.tokens || !b.positions ||
            !b.token_req || (b.n_want > 0 && (!logits || !b.want_rows)))
            return fail(IC_ERR_ARG, "the batch description", -1);
        const Workspace ws = layout(b);
        if (!workspace || workspace_bytes < (long long)ws.total) return fail(IC_ERR_ARG, "the workspace (too small)", -1);
        char* base = (char*)workspace;
        float* x = (float*)(base + ws.residual);
        void* normed = base + ws.normed;
        void* qkv = base + ws.qkv;
        void* attn_out = base + ws.attn_out;
        const int parts = ic_gemm_nt_residual_parts(d);
        int st;

        st = ic_embed(b.tokens, meta.embed_table, dt, x, T, d, meta.embed_scale, stream);
        if (st) return fail(st, "the embedding gather", -1);

        // what the residual stream still owes when a layer starts
        enum { NONE, BRANCH, DEFERRED, NORMED } owed = NONE;      // NORMED: the add and the whole norm are done, `normed` holds the rows
        const void* branch = nullptr;
        float branch_alpha = 0.f;
        Deferred def;

        const int last = meta.n_entries - 1;
        for (int i = 0; i <= last; ++i) {
            const IcRunEntry& e = entries[i];
            const IcLayer& L = layers[e.layer];
            const IcAttention& A = L.attention;
            if (e.group < 0 || e.group >= meta.n_groups || !b.group_tables[e.group]) return fail(IC_ERR_ARG, "the cache group of the entry", i);
            // the norm that whoever runs next applies first, if its rows may reach it half done
            const IcNorm* succ = nullptr;
            const float* succ_weight = nullptr;
            if (i < last) { succ = &layers[entries[i + 1].layer].mixer_norm; succ_weight = succ->weight; }
            else if (b.want_rows_identity) { succ = &meta.final_norm; succ_weight = meta.final_norm_scaled; }

            // ---- norm before the mixer -------------------------------------------------------------
            const Deferred* h_def = nullptr;
            if (owed == DEFERRED) h_def = &def;
            else if (owed == NORMED) {
            } else if (owed == NONE) {
                st = ic_rmsnorm(x, nullptr, L.mixer_norm.weight, normed, dt, T, d, L.mixer_norm.eps, 1.0f, stream);
                if (st) return fail(st, "the norm before attention", i);
            } else {
                st = ic_add_rmsnorm(x, branch, dt, branch_alpha, L.mixer_norm.weight, normed, dt, T, d, L.mixer_norm.eps, stream);
                if (st) return fail(st, "the residual add and norm before attention", i);
            }
            const void* h = h_def ? h_def->values : normed;

            // ---- attention: QKV, rotary, cache write -------------------------------------------------
            const int nkv = (A.shared_kv || !e.writes_cache) ? 0 : A.n_kv_heads;
            const int width = (A.n_heads + 2 * (A.shared_kv ? 0 : A.n_kv_heads)) * A.head_dim;
            const int* slots = b.group_slots[e.group];
            if (A.rot_dim > 0 && b.max_position >= A.max_positions) return fail(IC_ERR_ARG, "a position beyond the rotary tables", i);
            if (nkv > 0 && !slots) return fail(IC_ERR_ARG, "the cache slots of the entry's group", i);
            const bool fused_qkv = ic_rule_qkv_fused(dt, T, d, d, d, A.head_dim, A.rot_dim, nkv, h_def != nullptr) != 0;
            IcRowFactor rf{};
            if (h_def) rf = IcRowFactor{h_def->sumsq, h_def->parts, h_def->width, h_def->eps};
            if (fused_qkv) {
                st = ic_gemm_qkv_rope(h, A.w_qkv, qkv, T, d, d, d, width, b.positions, slots, A.cos, A.sin, e.k_cache, e.v_cache,
                                      A.n_heads, nkv, A.head_dim, ps, h_def ? &rf : nullptr, stream);
                if (st) return fail(st, "the QKV product with rotary and cache write", i);
            } else {
                st = linear(h, d, A.w_qkv, qkv, dt, T, width, d, 1.0f, h_def, lib_ws, lib_ws_bytes, stream);
                if (st) return fail(st, "the QKV product", i);
                if (A.rot_dim > 0 || nkv > 0) {
                    st = ic_rope_kv_write(qkv, dt, b.positions, A.rot_dim > 0 ? A.cos : nullptr, A.rot_dim > 0 ? A.sin : nullptr,
                                          nkv > 0 ? e.k_cache : nullptr, nkv > 0 ? e.v_cache : nullptr, nkv > 0 ? slots : nullptr, T,
                                          width, A.n_heads, nkv, A.head_dim, A.rot_dim, ps, stream);
                    if (st) return fail(st, "rotary and cache write", i);
                }
            }

            // ---- attention over the cache ---------------------------------------------------------------
            const int* tables = b.group_tables[e.group];
            const int bts = b.group_table_stride[e.group];
            const int ow = A.n_heads * A.head_dim;
            const int n_dec = b.n_decode_rows, n_tiles = b.n_prefill_tiles;
            const int attn = ic_rule_attention(dt, A.head_dim, ps, n_dec, n_tiles);
            const bool use_dec = (attn & IC_ATTN_SINGLE_TOKENS) != 0, use_pre = (attn & IC_ATTN_PORTIONS) != 0;
            if (attn == IC_ATTN_GENERAL) {
                st = ic_attn_generic(qkv, width, attn_out, ow, dt, e.k_cache, e.v_cache, tables, bts, b.token_req, b.positions, T,
                                     A.n_heads, A.n_kv_heads, A.head_dim, ps, A.softmax_scale, A.window, stream);
                if (st) return fail(st, "attention (general kernel)", i);
            } else {
                if (use_dec) {
                    const int n_split = splits_for(b, A);
                    st = ic_attn_decode(qkv, width, attn_out, ow, dt, e.k_cache, e.v_cache, tables, bts,
                                        b.decode_rows_identity ? nullptr : b.decode_rows, b.token_req, b.positions,
                                        (float*)(base + ws.part_acc), (float*)(base + ws.part_ml), n_dec, A.n_heads, A.n_kv_heads,
                                        A.head_dim, ps, A.softmax_scale, A.window, n_split, stream);
                    if (st) return fail(st, "attention of single tokens", i);
                }
                if (use_pre) {
                    int part_len = 0;
                    const int parts = tile_parts_for(b, A, &part_len);
                    st = ic_attn_prefill_split(qkv, width, attn_out, ow, dt, e.k_cache, e.v_cache, tables, bts, b.prefill_tiles,
                                               n_tiles, A.n_heads, A.n_kv_heads, A.head_dim, ps, A.softmax_scale, A.window, 0, parts,
                                               part_len, (float*)(base + ws.tile_parts),
                                               ic_attn_prefill_scratch_floats(n_tiles, A.n_heads, A.head_dim, parts),
                                               meta.attention_counters, stream);
                    if (st) return fail(st, "attention of prompt portions", i);
                }
            }

            // ---- O projection, residual add, norm before the feed-forward --------------------------------
            Deferred mid;
            const Deferred* g_def = nullptr;
            const int o_tail = ic_rule_tail(dt, T, d, ow, ow, ow);
            if (o_tail == IC_TAIL_SLICES) {
                st = tail_in_slices(attn_out, ow, A.w_o, (float*)(base + ws.tail_parts), x, L.residual_scale, L.ffn_norm.weight,
                                    L.ffn_norm.eps, normed, T, stream);
                if (st) return fail(st, "the O product in slices with residual add and norm", i);
            } else if (o_tail == IC_TAIL_SPLIT_NORM) {
                IcResidualNorm tail{x, d, L.ffn_norm.weight, L.residual_scale, (float*)(base + ws.mixer_sumsq), parts};
                st = ic_gemm_nt(attn_out, IC_BF16, A.w_o, IC_BF16, base + ws.mixer_tail, IC_BF16, T, d, ow, ow, ow, d, 1.0f, 2, nullptr,
                                &tail, stream);
                if (st) return fail(st, "the O product with residual add", i);
                mid = Deferred{base + ws.mixer_tail, (const float*)(base + ws.mixer_sumsq), parts, d, L.ffn_norm.eps};
                g_def = &mid;
            } else {
                st = linear(attn_out, ow, A.w_o, base + ws.mixer_out, dt, T, d, ow, 1.0f, nullptr, lib_ws, lib_ws_bytes, stream);
                if (st) return fail(st, "the O product", i);
                st = ic_add_rmsnorm(x, base + ws.mixer_out, dt, L.residual_scale, L.ffn_norm.weight, normed, dt, T, d, L.ffn_norm.eps, stream);
                if (st) return fail(st, "the residual add and norm before the feed-forward", i);
            }
            const void* g = g_def ? g_def->values : normed;

            // ---- feed-forward ----------------------------------------------------------------------------------
            const int di = L.ffn.intermediate;
            void* act = base + ws.act;
            if (ic_rule_gate_up_fused(dt, T, d, d, d, g_def != nullptr)) {
                IcRowFactor gf{};
                if (g_def) gf = IcRowFactor{g_def->sumsq, g_def->parts, g_def->width, g_def->eps};
                st = ic_gemm_nt(g, IC_BF16, L.ffn.w_gate_up, IC_BF16, act, IC_BF16, T, 2 * di, d, d, d, di, 1.0f, 1, g_def ? &gf : nullptr,
                                nullptr, stream);
                if (st) return fail(st, "the gate/up product with SwiGLU", i);
            } else {
                st = linear(g, d, L.ffn.w_gate_up, base + ws.gate_up, dt, T, 2 * di, d, 1.0f, nullptr, lib_ws, lib_ws_bytes, stream);
                if (st) return fail(st, "the gate/up product", i);
                st = ic_swiglu(base + ws.gate_up, act, dt, T, di, stream);
                if (st) return fail(st, "SwiGLU", i);
            }
            const int down_tail = succ ? ic_rule_tail(dt, T, d, di, di, di) : IC_TAIL_PLAIN;
            if (down_tail == IC_TAIL_SLICES) {
                st = tail_in_slices(act, di, L.ffn.w_down, (float*)(base + ws.tail_parts), x, L.residual_scale, succ_weight, succ->eps,
                                    normed, T, stream);
                if (st) return fail(st, "the down product in slices with residual add and norm", i);
                owed = NORMED;
            } else if (down_tail == IC_TAIL_SPLIT_NORM) {
                IcResidualNorm tail{x, d, succ_weight, L.residual_scale, (float*)(base + ws.ffn_sumsq), parts};
                st = ic_gemm_nt(act, IC_BF16, L.ffn.w_down, IC_BF16, base + ws.ffn_tail, IC_BF16, T, d, di, di, di, d, 1.0f, 2, nullptr,
                                &tail, stream);
                if (st) return fail(st, "the down product with residual add", i);
                def = Deferred{base + ws.ffn_tail, (const float*)(base + ws.ffn_sumsq), parts, d, succ->eps};
                owed = DEFERRED;
            } else {
                st = linear(act, di, L.ffn.w_down, base + ws.ffn_out, dt, T, d, di, 1.0f, nullptr, lib_ws, lib_ws_bytes, stream);
                if (st) return fail(st, "the down product", i);
                branch = base + ws.ffn_out;
                branch_alpha = L.residual_scale;
                owed = BRANCH;
            }
        }

        // ---- final norm and head, on the wanted rows only -----------------------------------------------------
        if (b.n_want == 0) return IC_OK;
        if (owed == NORMED) {        // every row in order, the final norm (with the logit scale in its weight) applied
            st = linear(normed, d, meta.head_weight, logits, IC_F32, T, meta.vocab, d, 1.0f, nullptr, lib_ws, lib_ws_bytes, stream);
            if (st) return fail(st, "the head product", -1);
            return IC_OK;
        }
        if (owed == DEFERRED) {      // every row in order, the final norm half done: its row factors go into the product
            st = linear(def.values, d, meta.head_weight, logits, IC_F32, T, meta.vocab, d, 1.0f, &def, lib_ws, lib_ws_bytes, stream);
            if (st) return fail(st, "the head product", -1);
            return IC_OK;
        }
        if (owed == BRANCH) {
            st = ic_residual_add(x, branch, dt, branch_alpha, (long long)T * d, stream);
            if (st) return fail(st, "the last residual add", -1);
        }
        void* head_in = base + ws.head_in;
        st = ic_rmsnorm(x, b.want_rows, meta.final_norm.weight, head_in, dt, b.n_want, d, meta.final_norm.eps, meta.logit_scale, stream);
        if (st) return fail(st, "the final norm", -1);
        st = linear(head_in, d, meta.head_weight, logits, IC_F32, b.n_want, meta.vocab, d, 1.0f, nullptr, lib_ws, lib_ws_bytes, stream);
        if (st) return fail(st, "the head product", -1);
        return IC_OK;
    }
};

IC_EXPORT const char* ic_decoder_create_error() { return g_create_error.c_str(); }

IC_EXPORT IcDecoder* ic_decoder_create(const IcDecoderMeta* meta, const IcLayer* layers, const IcRunEntry* entries) {
    g_create_error.clear();
    auto bad = [&](const char* what) -> IcDecoder* { g_create_error = what; return nullptr; };
    if (!meta || !layers || !entries) return bad("a null description");
    if (meta->dtype != IC_F32 && meta->dtype != IC_BF16) return bad("dtype must be 0 (float32) or 1 (bfloat16)");
    if (meta->hidden <= 0 || meta->vocab <= 0 || meta->page_size <= 0 || meta->n_layers <= 0 || meta->n_entries <= 0)
        return bad("hidden, vocab, page_size, n_layers and n_entries must be positive");
    if (meta->n_groups <= 0 || meta->n_groups > IC_MAX_CACHE_GROUPS) return bad("n_groups must lie in 1..8");
    if (!meta->embed_table || !meta->head_weight || !meta->final_norm.weight || !meta->final_norm_scaled)
        return bad("embedding table, head weight and final norm weights are needed");
    IcDecoder* d = new IcDecoder;
    d->meta = *meta;
    d->layers.assign(layers, layers + meta->n_layers);
    d->entries.assign(entries, entries + meta->n_entries);
    for (const IcLayer& l : d->layers) {
        const IcAttention& a = l.attention;
        const char* why = nullptr;
        if (a.n_heads <= 0 || a.n_kv_heads <= 0 || a.n_heads % a.n_kv_heads) why = "heads must be a positive multiple of kv heads";
        else if (a.head_dim <= 0 || a.head_dim % 16 || a.head_dim > 512) why = "head size must be a multiple of 16 up to 512";
        else if (a.rot_dim < 0 || a.rot_dim % 2 || a.rot_dim > a.head_dim) why = "rot_dim must be even and at most the head size";
        else if (a.rot_dim > 0 && (!a.cos || !a.sin || a.max_positions <= 0)) why = "rotary tables are needed";
        else if (!a.w_qkv || !a.w_o || !l.mixer_norm.weight || !l.ffn_norm.weight) why = "a layer lacks a weight";
        else if (l.ffn.intermediate <= 0 || !l.ffn.w_gate_up || !l.ffn.w_down) why = "the feed-forward lacks a size or a weight";
        if (why) { delete d; return bad(why); }
        d->max_qkv_width = std::max(d->max_qkv_width, (a.n_heads + 2 * (a.shared_kv ? 0 : a.n_kv_heads)) * a.head_dim);
        d->max_attn_width = std::max(d->max_attn_width, a.n_heads * a.head_dim);
        d->max_intermediate = std::max(d->max_intermediate, l.ffn.intermediate);
    }
    for (const IcRunEntry& e : d->entries) {
        if (e.layer < 0 || e.layer >= meta->n_layers || e.group < 0 || e.group >= meta->n_groups || !e.k_cache || !e.v_cache) {
            delete d;
            return bad("a run-order entry names no layer, no group or no cache planes");
        }
    }
    return d;
}

IC_EXPORT void ic_decoder_destroy(IcDecoder* decoder) { delete decoder; }

IC_EXPORT const char* ic_decoder_last_error(const IcDecoder* decoder) { return decoder ? decoder->error.c_str() : "no decoder"; }

IC_EXPORT long long ic_decoder_workspace_bytes(const IcDecoder* decoder, const IcStepBatch* batch) {
    if (!decoder || !batch || batch->n_tokens < 0 || batch->n_want < 0 || batch->n_decode_rows < 0) return -1;
    return (long long)decoder->layout(*batch).total;
}

IC_EXPORT int ic_decoder_forward(IcDecoder* decoder, const IcStepBatch* batch, void* workspace, long long workspace_bytes,
                                 void* library_workspace, long long library_workspace_bytes, float* logits, hipStream_t stream) {
    if (!decoder || !batch) return IC_ERR_ARG;
    return decoder->forward(*batch, workspace, workspace_bytes, library_workspace, library_workspace_bytes, logits, stream);
}

// ---- the key split of single-token rows --------------------------------------------------------------------------
// One split writes the result itself; more cost a second kernel (about 5 us), so short contexts are never split: up to
// 1,024 keys with one query head per kv head (a wave walks keys with vector instructions), up to 256 with grouped query
// heads on the matrix cores (its blocks walk 128 keys a round).  Beyond that, one head per kv head: few (row, kv head)
// pairs want about 1.75 blocks per compute unit but at least 384 keys a block; a middling number of pairs already draws
// the full bandwidth unsplit up to 2,048 keys; many pairs want about 3.4 blocks per unit.  Grouped heads: a wave has a
// whole 32-key tile in flight, so 128 / head size blocks per unit are enough and more only add partial results to merge.
// A split never gets fewer than 64 keys.
IC_EXPORT int ic_attn_decode_splits(int n_decode_rows, int n_heads, int n_kv_heads, int head_dim, int elem_bytes, int window,
                                    int max_context, int matrix_cores, int compute_units) {
    const int keys = std::max(1, window > 0 ? std::min(max_context, window) : max_context);
    const long long base = std::max(1LL, (long long)n_decode_rows * n_kv_heads);
    const double cu = compute_units > 0 ? compute_units : 256;
    const int s_max = std::max(1, std::min(64, keys / 64));
    if (matrix_cores) {
        // The grouped-query kernel: the same kind of model as below with constants of its own (fitted to 215 shapes of
        // 24:8 and 16:4 heads of 64, 32:2 and 32:8 of 128, 1..64 rows, 600..16,500 keys: 1.1 % from the best count on
        // average, worst 9 %; "128 / head size blocks a unit", which it replaces, 1.9 % and 32 %).  Up to 256 keys it
        // does not split.
        if (keys <= 256) return 1;
        const double stream_us = (double)base * keys * std::max(1, head_dim) * 2.0 * std::max(1, elem_bytes) / (6.42e6 * cu / 256.0);
        const double group = (double)std::max(1, n_heads) / std::max(1, n_kv_heads);
        int best = 1;
        double best_cost = 0.0;
        for (int s = 1; s <= s_max; ++s) {
            const double x = (double)base * s / cu;
            const double lost = 1.0 + (x > 1.0 ? 0.185 : 0.801) * (std::ceil(x) / x - 1.0);
            double cost = 1.882 + 5.201 / s + lost * stream_us;
            if (s > 1) cost += 6.632 + 0.153 * x * group;
            if (s == 1 || cost < best_cost) { best_cost = cost; best = s; }
        }
        return best;
    }
    // One head per wave: the split count with the least cost by a model of the two kernels' time in microseconds, fitted
    // to sweeps over 1..32 rows, 8..36 heads of 64 and 128, 600..16,500 keys with caches that do not fit the last-level
    // cache (on 370 shapes it loses 1.5 % against the best count on average, the rule of thumb it replaces 6 %):
    //   the bytes of keys and values at the rate the kernel streams them when every compute unit is busy,
    //   times what is lost when the last round of blocks fills the units only in part (x blocks a unit; less is lost
    //   below one block a unit, where a block's own latency sets the time),
    //   times what is lost when a block's share of the keys is not a whole number of its loop's 256-key rounds,
    //   plus a start-up cost that shrinks with shorter blocks, plus, with more than one split, the second kernel, its
    //   work per split and the partial results per block.
    const double stream_us = (double)base * keys * std::max(1, head_dim) * 2.0 * std::max(1, elem_bytes) / (6.631e6 * cu / 256.0);
    int best = 1;
    double best_cost = 0.0;
    for (int s = 1; s <= s_max; ++s) {
        const double x = (double)base * s / cu;
        double lost = 1.0 + (x > 1.0 ? 0.494 : 0.347) * (std::ceil(x) / x - 1.0);
        const int per = (keys + s - 1) / s;
        lost *= 1.0 + 0.299 * ((double)((per + 255) / 256 * 256) * s / keys - 1.0);
        double cost = 4.757 / s + lost * stream_us;
        if (s > 1) cost += 5.533 + 0.193 * s + 0.38 * x;
        if (s == 1 || cost < best_cost) { best_cost = cost; best = s; }
    }
    return best;
}

// ---- a batch given as host arrays ------------------------------------------------------------------------------------
namespace {

inline long long align4(long long n) { return (n + 3) & ~3LL; }

struct HostLayout {
    long long tokens, positions, token_req, want_rows, decode_rows, tiles, slots[IC_MAX_CACHE_GROUPS], tables[IC_MAX_CACHE_GROUPS], total;
    int n_want, n_decode, n_tiles, stride[IC_MAX_CACHE_GROUPS];
};

bool host_layout(const IcDecoder& dec, const IcHostBatch& b, HostLayout& h) {
    if (b.n_tokens <= 0 || b.n_requests <= 0 || !b.tokens || !b.req_lens || !b.req_pos || !b.tables || !b.table_len || b.tile_rows <= 0)
        return false;
    long long sum = 0;
    h.n_want = h.n_decode = h.n_tiles = 0;
    for (int r = 0; r < b.n_requests; ++r) {
        const int n = b.req_lens[r];
        if (n <= 0 || b.req_pos[r] < 0) return false;
        sum += n;
        if (b.want_count) h.n_want += b.want_count[r];
        if (n == 1) ++h.n_decode;
        else h.n_tiles += (n + b.tile_rows - 1) / b.tile_rows;
    }
    if (sum != b.n_tokens || (h.n_want > 0 && !b.want)) return false;
    const long long T = b.n_tokens;
    long long o = 0;
    auto take = [&](long long n) { const long long at = o; o += align4(n); return at; };
    h.tokens = take(T); h.positions = take(T); h.token_req = take(T);
    h.want_rows = take(h.n_want); h.decode_rows = take(h.n_decode); h.tiles = take(4LL * h.n_tiles);
    const int ps = dec.meta.page_size;
    for (int g = 0; g < dec.meta.n_groups; ++g) {
        int longest = 1;
        for (int r = 0; r < b.n_requests; ++r) {
            const int len = b.table_len[g * b.n_requests + r];
            if (len < (b.req_pos[r] + b.req_lens[r] + ps - 1) / ps || !b.tables[g * b.n_requests + r]) return false;
            longest = std::max(longest, len);
        }
        h.stride[g] = longest;
        h.slots[g] = take(T);
        h.tables[g] = take((long long)b.n_requests * longest);
    }
    h.total = o;
    return true;
}

}  // namespace

IC_EXPORT long long ic_decoder_step_ints(const IcDecoder* decoder, const IcHostBatch* batch) {
    HostLayout h;
    if (!decoder || !batch || !host_layout(*decoder, *batch, h)) return -1;
    return h.total;
}

IC_EXPORT int ic_decoder_pack(const IcDecoder* decoder, const IcHostBatch* batch, int* staging, const int* device_ints,
                              long long n_ints, IcStepBatch* out) {
    HostLayout h;
    if (!decoder || !batch || !staging || !device_ints || !out || !host_layout(*decoder, *batch, h) || n_ints < h.total) return IC_ERR_ARG;
    const IcHostBatch& b = *batch;
    const int ps = decoder->meta.page_size, R = b.n_requests;
    struct Row { int pos, row; };
    struct Tile { int req, row, rows, pos; };
    std::vector<Row> dec;
    std::vector<Tile> tiles;
    dec.reserve(h.n_decode);
    tiles.reserve(h.n_tiles);
    int row0 = 0, w = 0, max_pos = 0, max_ctx = 0;
    const int* want = b.want;
    bool identity = h.n_want == b.n_tokens;
    for (int r = 0; r < R; ++r) {
        const int n = b.req_lens[r], p0 = b.req_pos[r];
        for (int i = 0; i < n; ++i) {
            staging[h.tokens + row0 + i] = b.tokens[row0 + i];
            staging[h.positions + row0 + i] = p0 + i;
            staging[h.token_req + row0 + i] = r;
        }
        const int nw = b.want_count ? b.want_count[r] : 0;
        for (int i = 0; i < nw; ++i) {
            if (want[i] < 0 || want[i] >= n) return IC_ERR_ARG;
            identity = identity && (row0 + want[i] == w);
            staging[h.want_rows + w++] = row0 + want[i];
        }
        want += nw;
        if (n == 1) { dec.push_back(Row{p0, row0}); max_ctx = std::max(max_ctx, p0 + 1); }
        else for (int o = 0; o < n; o += b.tile_rows) tiles.push_back(Tile{r, row0 + o, std::min(b.tile_rows, n - o), p0 + o});
        max_pos = std::max(max_pos, p0 + n - 1);
        for (int g = 0; g < decoder->meta.n_groups; ++g) {
            const int* table = b.tables[g * R + r];
            const int len = b.table_len[g * R + r], stride = h.stride[g];
            for (int i = 0; i < n; ++i) staging[h.slots[g] + row0 + i] = table[(p0 + i) / ps] * ps + (p0 + i) % ps;
            int* dst = staging + h.tables[g] + (long long)r * stride;
            for (int j = 0; j < len; ++j) dst[j] = table[j] > 0 ? table[j] : 0;     // pages given back are never read; keep the index valid
            for (int j = len; j < stride; ++j) dst[j] = 0;
        }
        row0 += n;
    }
    // tiles that see the most keys go first, so the longest blocks do not form the tail; likewise the single tokens,
    // unless all rows are single tokens and the kernel takes the rows as they lie
    std::stable_sort(tiles.begin(), tiles.end(), [](const Tile& a, const Tile& c) { return a.pos + a.rows > c.pos + c.rows; });
    if ((int)dec.size() < b.n_tokens) std::stable_sort(dec.begin(), dec.end(), [](const Row& a, const Row& c) { return a.pos > c.pos; });
    for (size_t i = 0; i < dec.size(); ++i) staging[h.decode_rows + i] = dec[i].row;
    for (size_t i = 0; i < tiles.size(); ++i) {
        int* t = staging + h.tiles + 4 * i;
        t[0] = tiles[i].req; t[1] = tiles[i].row; t[2] = tiles[i].rows; t[3] = tiles[i].pos;
    }
    IcStepBatch s{};
    s.n_tokens = b.n_tokens; s.n_requests = R; s.n_want = h.n_want; s.n_decode_rows = (int)dec.size(); s.n_prefill_tiles = (int)tiles.size();
    s.want_rows_identity = identity ? 1 : 0;
    s.decode_rows_identity = (int)dec.size() == b.n_tokens ? 1 : 0;
    s.max_position = max_pos;
    s.max_context = max_ctx ? ic_rule_context_bucket(max_ctx) : 0;
    s.fixed_decode_splits = b.fixed_decode_splits;
    s.tokens = device_ints + h.tokens; s.positions = device_ints + h.positions; s.token_req = device_ints + h.token_req;
    s.want_rows = device_ints + h.want_rows; s.decode_rows = device_ints + h.decode_rows; s.prefill_tiles = device_ints + h.tiles;
    for (int g = 0; g < decoder->meta.n_groups; ++g) {
        s.group_slots[g] = device_ints + h.slots[g];
        s.group_tables[g] = device_ints + h.tables[g];
        s.group_table_stride[g] = h.stride[g];
    }
    *out = s;
    return IC_OK;
}

IC_EXPORT int ic_decoder_step(IcDecoder* decoder, const IcHostBatch* batch, int* staging, int* device_ints, long long n_ints,
                              void* workspace, long long workspace_bytes, void* library_workspace, long long library_workspace_bytes,
                              float* logits, IcStepBatch* laid_out, hipStream_t stream) {
    IcStepBatch s;
    int st = ic_decoder_pack(decoder, batch, staging, device_ints, n_ints, &s);
    if (st) return decoder ? decoder->fail(st, "laying out the batch", -1) : st;
    const long long need = ic_decoder_step_ints(decoder, batch);
    hipError_t e = hipMemcpyAsync(device_ints, staging, (size_t)need * sizeof(int), hipMemcpyHostToDevice, stream);
    if (e != hipSuccess) return decoder->fail((int)e, "the copy of the step's integers", -1);
    if (laid_out) *laid_out = s;
    return decoder->forward(s, workspace, workspace_bytes, library_workspace, library_workspace_bytes, logits, stream);
}
