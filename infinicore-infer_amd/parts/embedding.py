"""Token embedding and output head.

Embedding: x = E[token] * scale_emb (scripts/jiuge.py:193-197; gather at
src/models/jiuge/jiuge.cpp:164-168).  The scale is applied at gather time, so a
tied table is held once.  Head: logits = (norm(x) * logit_scale) W^T in
float32 out (jiuge.py:198-207, jiuge.cpp:262-264,270-278), only for the rows
that are asked for.  Which tensor backs which table follows the reference: the
embedding falls back to lm_head.weight and the head to model.embed_tokens.weight
when its own tensor is absent (jiuge.py:182-191).
"""
import torch

from ..kernels import ops
from ..weights.loader import WeightSpec
from .base import DeferredRows, Part, register_part
from .linear import linear


@register_part("embedding", "embedding")
class Embedding(Part):
    graph_safe = True

    category = "embedding"

    def __init__(self, name, runtime, vocab_size: int, hidden_size: int, scale: float = 1.0,
                 fallback_name=None):
        super().__init__(name, runtime)
        self.vocab_size, self.hidden_size = vocab_size, hidden_size
        self.scale = float(scale)
        self.fallback = fallback_name + "weight" if fallback_name else None
        self.table = None

    def weight_specs(self):
        return {self.name + "weight": WeightSpec((self.vocab_size, self.hidden_size), "matrix", self.fallback)}

    def load_weights(self, tensors):
        self.table = tensors[self.name + "weight"]

    def forward(self, tokens, x):
        return ops.embed(tokens, self.table, x, self.scale)

    def native_desc(self):
        """(table address, scale) for the native step function."""
        t = self.table
        if not (self._forward_is(Embedding) and t is not None and t.is_cuda and t.dtype == self.runtime.dtype
                and t.is_contiguous()):
            return None
        return (t.data_ptr(), self.scale)


class _ScaledNorm:
    """(weight, eps) of a norm whose weight already carries the head's scale."""

    def __init__(self, weight, eps):
        self._d = (weight, eps)

    def deferred(self):
        return self._d


@register_part("head", "lm_head")
class LMHead(Part):
    graph_safe = True
    accepts_deferred = True

    category = "head"

    def __init__(self, name, runtime, vocab_size: int, hidden_size: int, logit_scale: float = 1.0,
                 fallback_name=None, tied: bool = False):
        super().__init__(name, runtime)
        self.vocab_size, self.hidden_size = vocab_size, hidden_size
        self.logit_scale = float(logit_scale)
        self.fallback = fallback_name + "weight" if fallback_name else None
        self.tied = bool(tied) and self.fallback is not None
        self.weight = None
        self._scaled_norms = {}

    def weight_specs(self):
        return {self.name + "weight": WeightSpec((self.vocab_size, self.hidden_size), "matrix", self.fallback,
                                                 tied=self.tied)}

    def load_weights(self, tensors):
        self.weight = tensors[self.name + "weight"]
        self._scaled_norms = {}

    def deferred_norm(self, final_norm):
        """The final norm as the last block's successor when its rows reach the head half done: its
        weight times the logit scale, so that the scale enters before the rounding to the compute
        dtype exactly as on the other path (``out_scale`` of the norm kernel; the reference scales
        the norm's weight, scripts/jiuge.py:198-201).  None when the norm cannot be split."""
        d = final_norm.deferred()
        if d is None:
            return None
        key = id(final_norm)
        if key not in self._scaled_norms:
            self._scaled_norms[key] = _ScaledNorm((d[0] * self.logit_scale).contiguous(), d[1])
        return self._scaled_norms[key]

    def native_desc(self):
        """(weight address, logit scale) for the native step function."""
        w = self.weight
        if not (self._forward_is(LMHead) and w is not None and w.is_cuda and w.dtype == self.runtime.dtype
                and w.is_contiguous()):
            return None
        return (w.data_ptr(), self.logit_scale)

    def forward(self, x, rows, final_norm, ctx):
        """Float32 logits [len(rows), vocab] of the residual rows ``rows``."""
        if isinstance(x, DeferredRows):
            # every row in order, the final norm half done: its row factors go into the product
            logits = ctx.ws.buffer("logits", (x.shape[0], self.vocab_size), torch.float32)
            return linear(x, self.weight, logits, self.runtime.gemm_impl, ws=ctx.ws)     # the scale is in x (deferred_norm)
        n = rows.numel()
        h = ctx.ws.buffer("head_in", (n, self.hidden_size), self.runtime.dtype)
        final_norm.forward(x, h, rows=rows, out_scale=self.logit_scale)
        logits = ctx.ws.buffer("logits", (n, self.vocab_size), torch.float32)
        linear(h, self.weight, logits, self.runtime.gemm_impl, ws=ctx.ws)
        return logits
