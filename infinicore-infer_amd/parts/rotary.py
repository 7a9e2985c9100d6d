"""Rotary position encoding, fused with the write of keys and values into the
paged cache.

Angles: pos / theta^(j / (dh/2)) for pair j (src/models/jiuge/jiuge_weight.hpp:134-186).
The reference rotates adjacent pairs of q_proj/k_proj rows that it permuted on
the host (scripts/jiuge.py:217-227); that equals rotating pairs (j, j + dh/2)
of the checkpoint's own row order, which is what the kernel does, so weights
load unpermuted.  Tables are built in float64 and held in float32.

Long-context scaling ("longrope", not in the reference): each pair's frequency
is divided by a factor from the long array when the checkpoint's context
(max_position_embeddings, not a serving cap on it) exceeds the original one, else
from the short array; cos and sin are multiplied by
sqrt(1 + ln(ratio) / ln(original)) when ratio = context / original > 1.
"""
import math

import torch

from ..kernels import ops
from .base import DeferredRows, PositionEncoding, register_part


def rotary_tables(head_dim, theta, max_positions, scaling=None, rot_dim=None, model_max_positions=None):
    """cos and sin [max_positions, rot/2] in float32.  ``max_positions`` is only the tables' length;
    long-context scaling (which factor array, the magnitude) follows ``model_max_positions``, the
    checkpoint's own context length, so a serving cap on the context changes no value."""
    rot = head_dim if rot_dim is None else rot_dim
    if model_max_positions is None:
        model_max_positions = max_positions
    half = rot // 2
    j = torch.arange(half, dtype=torch.float64)
    inv_freq = 1.0 / torch.pow(torch.tensor(float(theta), dtype=torch.float64), j / half)
    magnitude = 1.0
    if scaling:
        orig = int(scaling["original_max_position_embeddings"])
        ratio = model_max_positions / orig
        if ratio > 1.0:
            factors = scaling["long_factor"]
            magnitude = math.sqrt(1.0 + math.log(ratio) / math.log(orig))
        else:
            factors = scaling["short_factor"]
        inv_freq = inv_freq / torch.tensor(factors, dtype=torch.float64)
    ang = torch.arange(max_positions, dtype=torch.float64)[:, None] * inv_freq[None, :]
    return (torch.cos(ang) * magnitude).to(torch.float32), (torch.sin(ang) * magnitude).to(torch.float32)


_TABLES = {}


@register_part("position_encoding", "rotary")
class Rotary(PositionEncoding):
    graph_safe = True

    def __init__(self, name, runtime, head_dim: int, theta: float, max_positions: int, scaling=None,
                 rot_dim=None, model_max_positions=None):
        super().__init__(name, runtime)
        self.head_dim = head_dim
        self.rot_dim = head_dim if rot_dim is None else rot_dim
        if self.rot_dim % 2 or self.rot_dim > head_dim:
            raise ValueError("rotary: rot_dim must be even and at most head_dim")
        self.max_positions = max_positions
        key = (head_dim, float(theta), max_positions, repr(scaling), self.rot_dim, model_max_positions,
               str(runtime.device))
        if key not in _TABLES:            # layers with the same parameters share one pair of tables
            cos, sin = rotary_tables(head_dim, theta, max_positions, scaling, self.rot_dim, model_max_positions)
            _TABLES[key] = (cos.to(runtime.device).contiguous(), sin.to(runtime.device).contiguous())
        self.cos, self.sin = _TABLES[key]

    def position_limit(self):
        return self.max_positions

    def native_rotary(self):
        """(rot_dim, table rows, cos address, sin address) for the native step function."""
        if type(self).rotate_and_store is not Rotary.rotate_and_store or \
                type(self).project_rotate_store is not Rotary.project_rotate_store or not self.cos.is_cuda:
            return None
        return (self.rot_dim, self.max_positions, self.cos.data_ptr(), self.sin.data_ptr())

    def rotate_and_store(self, qkv, ctx, cache, n_heads, n_kv_heads, head_dim):
        if ctx.max_position >= self.max_positions:
            raise ValueError("position %d is beyond the rotary tables (%d)" % (ctx.max_position, self.max_positions))
        k, v = (cache.k, cache.v) if n_kv_heads > 0 else (None, None)
        ops.rope_kv_write(qkv, ctx.positions, self.cos, self.sin, k, v,
                          cache.slots if n_kv_heads > 0 else None,
                          n_heads, n_kv_heads, head_dim, self.rot_dim, ctx.page_size)


    def project_rotate_store(self, h, w_qkv, qkv, ctx, cache, n_heads, n_kv_heads, head_dim) -> bool:
        """Few rows in bfloat16 with full rotary: the projection kernel rotates and writes the cache."""
        rt = self.runtime
        row_factor = None
        if isinstance(h, DeferredRows):
            h, row_factor = h.values, h.row_factor()
        if (rt.gemm_impl != "auto" or h.dtype != w_qkv.dtype or h.dtype != qkv.dtype
                or not ops.rule_qkv_fused(h.dtype, h.shape[0], h, w_qkv, head_dim, self.rot_dim, n_kv_heads,
                                          row_factor is not None)):
            return False
        if ctx.max_position >= self.max_positions:
            raise ValueError("position %d is beyond the rotary tables (%d)" % (ctx.max_position, self.max_positions))
        ops.gemm_qkv_rope(h, w_qkv, qkv, ctx.positions, cache.slots, self.cos, self.sin, cache.k, cache.v,
                          n_heads, n_kv_heads, head_dim, ctx.page_size, row_factor=row_factor)
        return True


@register_part("position_encoding", "none")
class NoPositionEncoding(PositionEncoding):
    """No rotation: only the cache write."""
    graph_safe = True

    def __init__(self, name, runtime, **_):
        super().__init__(name, runtime)

    def native_rotary(self):
        if type(self).rotate_and_store is not NoPositionEncoding.rotate_and_store:
            return None
        return (0, 0, None, None)

    def rotate_and_store(self, qkv, ctx, cache, n_heads, n_kv_heads, head_dim):
        if n_kv_heads > 0:
            ops.rope_kv_write(qkv, ctx.positions, None, None, cache.k, cache.v, cache.slots,
                              n_heads, n_kv_heads, head_dim, 0, ctx.page_size)
