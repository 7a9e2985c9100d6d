"""Softmax attention over the paged cache (MHA or grouped-query).

Per layer the reference does (src/models/jiuge/jiuge.cpp:200-236): fused QKV
projection, rotary on q and k heads, append k and v to the cache, scores
(1/sqrt(dh)) Q K^T over keys 0..t-1, causal softmax aligned to the bottom right,
P V, output projection.  Query head h uses key/value head h // (nh/nkvh)
(jiuge.cpp:210-213).  Here the scores never reach memory: one of three kernels
walks the cache with a float32 running softmax,
  * a split-key kernel for rows that are a request's single new token,
  * a matrix-core kernel for prompt portions (head size 64 or 128; bfloat16, or true float32 with
    float32 matrix instructions),
  * the general kernel for everything else.
"""
import torch

from ..kernels import ops
from ..weights.loader import WeightSpec
from .base import CacheNeed, DeferredRows, Mixer, build_part, register_part
from .linear import linear, linear_tail


@register_part("mixer", "attention")
class Attention(Mixer):
    graph_safe = True
    accepts_deferred = True
    fuses_tail = True

    def __init__(self, name, runtime, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int,
                 softmax_scale: float, position_encoding, window=None, shared_kv: bool = False):
        super().__init__(name, runtime)
        if num_heads % num_kv_heads:
            raise ValueError("attention: %d heads are not a multiple of %d kv heads" % (num_heads, num_kv_heads))
        if head_dim % 16:
            raise ValueError("attention: head size %d is not a multiple of 16" % head_dim)
        if head_dim > 512:
            raise ValueError("attention: head size %d above 512" % head_dim)
        self.hidden_size = hidden_size
        self.nh, self.nkvh, self.dh = num_heads, num_kv_heads, head_dim
        self.scale = float(softmax_scale)
        self.window = int(window) if window else 0
        self.shared_kv = bool(shared_kv)          # reads another entry's cache: projects q only
        self.pos_enc = position_encoding if not hasattr(position_encoding, "kind") \
            else build_part("position_encoding", position_encoding, runtime)
        self.w_qkv = None
        self.w_o = None

    def sub_parts(self):
        return (self.pos_enc,)

    def cache_need(self):
        return CacheNeed("kv", self.nkvh, self.dh, self.window or None)

    def portion_tile_rows(self):
        return ops.attention_prefill_tile_rows()

    # ---- weights: names of scripts/jiuge.py:45-63 ------------------------------
    def weight_specs(self):
        n = self.name
        pack = None if self.shared_kv else n + "qkv_proj.packed"
        specs = {
            n + "q_proj.weight": WeightSpec((self.nh * self.dh, self.hidden_size), pack=pack and (pack, 0)),
            n + "o_proj.weight": WeightSpec((self.hidden_size, self.nh * self.dh)),
        }
        if not self.shared_kv:
            specs[n + "k_proj.weight"] = WeightSpec((self.nkvh * self.dh, self.hidden_size), pack=(pack, 1))
            specs[n + "v_proj.weight"] = WeightSpec((self.nkvh * self.dh, self.hidden_size), pack=(pack, 2))
        return specs

    def load_weights(self, tensors):
        n = self.name
        names = ["q_proj.weight"] + ([] if self.shared_kv else ["k_proj.weight", "v_proj.weight"])
        mats = [tensors[n + s] for s in names]
        # rows [Q; K; V] of one fused projection (jiuge.py:237-239), unpermuted.  The loader lays the
        # three out one after the other and hands out their concatenation; otherwise copy them together.
        packed = tensors.get(n + "qkv_proj.packed")
        if packed is not None:
            self.w_qkv = packed
        else:
            if len({m.dtype for m in mats}) > 1:
                mats = [m.to(torch.float32) for m in mats]
            self.w_qkv = torch.cat(mats, dim=0).contiguous() if len(mats) > 1 else mats[0]
        self.w_o = tensors[n + "o_proj.weight"]

    def native_desc(self):
        from ..kernels.lib import IcAttention
        rot = getattr(self.pos_enc, "native_rotary", lambda: None)()
        ws = (self.w_qkv, self.w_o)
        if not (self._forward_is(Attention) and type(self)._attend is Attention._attend and rot is not None
                and all(w is not None and w.is_cuda and w.dtype == self.runtime.dtype and w.is_contiguous() for w in ws)):
            return None
        return IcAttention(self.nh, self.nkvh, self.dh, self.window, int(self.shared_kv), rot[0], rot[1], self.scale,
                           rot[2], rot[3], self.w_qkv.data_ptr(), self.w_o.data_ptr())

    # ---- forward ---------------------------------------------------------------------
    def forward(self, h, ctx, cache, tail=None):
        rt = self.runtime
        T = h.shape[0]
        nkv = 0 if (self.shared_kv or not cache.writes) else self.nkvh
        width = (self.nh + 2 * (0 if self.shared_kv else self.nkvh)) * self.dh
        qkv = ctx.ws.buffer("qkv", (T, width), rt.dtype)
        if not self.pos_enc.project_rotate_store(h, self.w_qkv, qkv, ctx, cache, self.nh, nkv, self.dh):
            linear(h, self.w_qkv, qkv, rt.gemm_impl, ws=ctx.ws)
            self.pos_enc.rotate_and_store(qkv, ctx, cache, self.nh, nkv, self.dh)
        out = ctx.ws.buffer("attn_out", (T, self.nh * self.dh), rt.dtype)
        self._attend(qkv, out, ctx, cache)
        fused = linear_tail(out, self.w_o, tail, ctx.ws, "mixer_tail", rt.gemm_impl)
        if fused is not None:
            return fused
        y = ctx.ws.buffer("mixer_out", (T, self.hidden_size), rt.dtype)
        linear(out, self.w_o, y, rt.gemm_impl, ws=ctx.ws)
        return y

    def _key_splits(self, ctx) -> int:
        """How many ways to split the keys of single-token rows: the kernel library's rule
        (ic_attn_decode_splits, from sweeps on MI355X with a cold cache), so that steps issued from
        Python and from native code split alike.  The layers of a model mostly ask the same question,
        so the answer is kept in the step's memo."""
        if ctx.fixed_decode_splits is not None:
            return ctx.fixed_decode_splits
        rt = self.runtime
        key = (ctx.n_decode_rows, self.nh, self.nkvh, self.dh, 2 if rt.dtype == torch.bfloat16 else 4, self.window,
               ctx.max_context, int(ops.attention_decode_on_matrix_cores(rt.dtype, self.nh, self.nkvh)), ctx.cu_count)
        memo = ctx.memo.get("attention_key_splits")
        if memo is None or memo[0] != key:
            memo = ctx.memo["attention_key_splits"] = (key, ops.attention_decode_splits(*key))
        return memo[1]

    def _attend(self, q, out, ctx, cache):
        rt = self.runtime
        args = (self.nh, self.nkvh, self.dh, ctx.page_size)
        n_dec, n_tiles = ctx.n_decode_rows, ctx.n_prefill_tiles
        how = ops.ATTN_GENERAL
        if rt.attention_impl == "auto":
            how = ops.rule_attention(rt.dtype, self.dh, ctx.page_size, n_dec, n_tiles)
        use_dec, use_pre = bool(how & ops.ATTN_SINGLE_TOKENS), bool(how & ops.ATTN_PORTIONS)
        if how == ops.ATTN_GENERAL:
            ops.attention_generic(q, out, cache.k, cache.v, cache.block_tables, ctx.token_req, ctx.positions,
                                  *args, self.scale, self.window)
            return
        if use_dec:
            n_split = self._key_splits(ctx)
            part_acc = ctx.ws.buffer("attn_part_acc", (n_dec * self.nh * n_split * self.dh,), torch.float32)
            part_ml = ctx.ws.buffer("attn_part_ml", (n_dec * self.nh * n_split * 2,), torch.float32)
            ops.attention_decode(q, out, cache.k, cache.v, cache.block_tables,
                                 None if ctx.decode_rows_identity else ctx.decode_rows, n_dec,
                                 ctx.token_req, ctx.positions, part_acc, part_ml, *args, self.scale,
                                 self.window, n_split)
        if use_pre:
            # few blocks and long walks over the keys: the tiles' walks are cut into parts (the library's rule)
            parts, part_len = ops.attention_prefill_parts_of_step(rt.dtype, n_tiles, self.nh, self.dh, ctx.max_position, self.window, ctx.cu_count)
            scratch = counters = None
            if parts > 1:
                scratch = ctx.ws.buffer("attn_tile_parts", (ops.attention_prefill_scratch_floats(n_tiles, self.nh, self.dh, parts),),
                                        torch.float32)
                counters = ctx.ws.zeroed("attn_tile_arrivals", (ops.attention_prefill_counter_ints(),), torch.int32)
            ops.attention_prefill(q, out, cache.k, cache.v, cache.block_tables, ctx.prefill_tiles, n_tiles,
                                  *args, self.scale, self.window, parts=parts, part_len=part_len, scratch=scratch,
                                  counters=counters)
