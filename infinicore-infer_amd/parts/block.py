"""Pre-norm residual block: x += a * mixer(norm1(x)); x += a * ffn(norm2(x)),
with a = scale_depth / sqrt(num_layers) (scripts/jiuge.py:109-114; the
reference folds it into o_proj and down_proj, jiuge.py:284-299,335-350, here it
is a float32 factor of the residual add).  The layer body is
src/models/jiuge/jiuge.cpp:195-258.

The residual stream is float32.  Each add is fused with the norm that follows
it: the block leaves its last add pending for whoever normalises next.
"""
from .base import Block, register_part


@register_part("block", "prenorm_residual")
class PreNormResidualBlock(Block):
    graph_safe = True

    def __init__(self, name, runtime, mixer, mixer_norm, feed_forward, feed_forward_norm,
                 residual_scale: float = 1.0):
        super().__init__(name, runtime, mixer, mixer_norm, feed_forward, feed_forward_norm)
        self.residual_scale = float(residual_scale)

    def forward(self, x, pending, ctx, cache):
        h = ctx.ws.buffer("normed", tuple(x.shape), self.runtime.dtype)
        if pending is None:
            self.mixer_norm.forward(x, h)
        else:
            self.mixer_norm.forward_add(x, pending[0], pending[1], h)
        y = self.mixer.forward(h, ctx, cache)
        self.feed_forward_norm.forward_add(x, y, self.residual_scale, h)
        y = self.feed_forward.forward(h, ctx)
        return (y, self.residual_scale)
