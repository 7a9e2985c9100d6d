"""Pre-norm residual block: x += a * mixer(norm1(x)); x += a * ffn(norm2(x))
(the second half only when the layer has a feed-forward: a stack of mixers alone leaves it out),
with a = scale_depth / sqrt(num_layers) (scripts/jiuge.py:109-114; the
reference folds it into o_proj and down_proj, jiuge.py:284-299,335-350, here it
is a float32 factor of the residual add).  The layer body is
src/models/jiuge/jiuge.cpp:195-258.

The residual stream is float32.  Each add is fused with the norm that follows
it: the block leaves its last add pending for whoever normalises next.  For
few rows the add and the norm go further, into the products on either side
(``ResidualTail`` / ``DeferredRows``): then a layer is six kernels, not eight.
"""
from .base import Block, DeferredRows, ResidualTail, register_part


@register_part("block", "prenorm_residual")
class PreNormResidualBlock(Block):
    graph_safe = True
    fuses_successor = True

    def __init__(self, name, runtime, mixer=None, mixer_norm=None, feed_forward=None, feed_forward_norm=None,
                 residual_scale: float = 1.0):
        super().__init__(name, runtime, mixer, mixer_norm, feed_forward, feed_forward_norm)
        if mixer is None or mixer_norm is None:
            raise ValueError("block %s: a pre-norm residual block needs a mixer and its norm" % name)
        if (feed_forward is None) != (feed_forward_norm is None):
            raise ValueError("block %s: a feed-forward and its norm come together, or neither" % name)
        self.residual_scale = float(residual_scale)

    def entry_norm(self):
        """The norm applied to the incoming stream, if the mixer can take its rows half done."""
        return self.mixer_norm if getattr(self.mixer, "accepts_deferred", False) else None

    def _tail(self, producer, consumer_ok, norm, x):
        """The request to fuse (add, norm) into the producer's last projection, when all three agree."""
        if not (getattr(producer, "fuses_tail", False) and consumer_ok and norm is not None):
            return None
        d = norm.deferred()
        return None if d is None else ResidualTail(x, self.residual_scale, d[0], d[1])

    def native_desc(self):
        """The layer for the native step function, when it is this arrangement of parts that all have
        a native description themselves (attention, SwiGLU, RMS norms)."""
        from ..kernels.lib import IcAttention, IcLayer, IcNorm, IcSwiGLU
        if not self._forward_is(PreNormResidualBlock) or self.feed_forward is None:
            return None
        descs = [p.native_desc() for p in (self.mixer_norm, self.mixer, self.feed_forward_norm, self.feed_forward)]
        if not (isinstance(descs[0], IcNorm) and isinstance(descs[1], IcAttention) and isinstance(descs[2], IcNorm)
                and isinstance(descs[3], IcSwiGLU)):
            return None
        return IcLayer(descs[0], descs[1], descs[2], descs[3], self.residual_scale)

    def forward(self, x, pending, ctx, cache, successor=None):
        if isinstance(pending, DeferredRows):
            h = pending                               # the add is done; the mixer applies the row factors
        else:
            h = ctx.ws.buffer("normed", tuple(x.shape), self.runtime.dtype)
            if pending is None:
                self.mixer_norm.forward(x, h)
            else:
                self.mixer_norm.forward_add(x, pending[0], pending[1], h)
        if self.feed_forward is None:                 # a layer of a mixer alone: its add is what the layer leaves owed
            tail = self._tail(self.mixer, True, successor, x)
            y = self.mixer.forward(h, ctx, cache, tail=tail) if tail is not None else self.mixer.forward(h, ctx, cache)
            return y if isinstance(y, DeferredRows) else (y, self.residual_scale)
        tail = self._tail(self.mixer, getattr(self.feed_forward, "accepts_deferred", False), self.feed_forward_norm, x)
        y = self.mixer.forward(h, ctx, cache, tail=tail) if tail is not None else self.mixer.forward(h, ctx, cache)
        if isinstance(y, DeferredRows):
            h = y
        else:
            h = ctx.ws.buffer("normed", tuple(x.shape), self.runtime.dtype)
            self.feed_forward_norm.forward_add(x, y, self.residual_scale, h)
        tail = self._tail(self.feed_forward, True, successor, x)
        y = self.feed_forward.forward(h, ctx, tail=tail) if tail is not None else self.feed_forward.forward(h, ctx)
        if isinstance(y, DeferredRows):
            return y
        return (y, self.residual_scale)
