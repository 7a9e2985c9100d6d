"""RMSNorm: y = x * rsqrt(mean(x^2) + eps) * w, computed in float32 on the
float32 residual stream (call sites src/models/jiuge/jiuge.cpp:198,246,262;
eps = rms_norm_eps, scripts/jiuge.py:132; weights kept in float32,
scripts/jiuge.py:146,209-215)."""
import torch

from ..kernels import ops
from ..weights.loader import WeightSpec
from .base import Norm, register_part


@register_part("norm", "rmsnorm")
class RMSNorm(Norm):
    graph_safe = True

    def __init__(self, name, runtime, size: int, eps: float):
        super().__init__(name, runtime)
        self.size = size
        self.eps = float(eps)
        self.weight = None

    def weight_specs(self):
        return {self.name + "weight": WeightSpec((self.size,), "vector")}

    def load_weights(self, tensors):
        self.weight = tensors[self.name + "weight"]

    def forward(self, x, out, rows=None, out_scale: float = 1.0):
        return ops.rmsnorm(x, self.weight, out, self.eps, out_scale, rows)

    def forward_add(self, x, y, alpha, out):
        return ops.add_rmsnorm(x, y, alpha, self.weight, out, self.eps)

    def deferred(self):
        return (self.weight, self.eps)

    def native_desc(self):
        from ..kernels.lib import IcNorm
        w = self.weight
        if not (self._forward_is(RMSNorm) and w is not None and w.is_cuda and w.dtype == torch.float32
                and w.is_contiguous()):
            return None
        return IcNorm(w.data_ptr(), self.eps)
