"""Dense SwiGLU feed-forward: down( up(h) * silu(gate(h)) ).

The reference fuses gate and up into one projection with rows [gate; up]
(scripts/jiuge.py:311-323), applies swiglu(out=gate, up, gate)
(src/models/jiuge/jiuge.cpp:247-248) and projects down (jiuge.cpp:249).  No
biases.  The activation is computed in float32 inside the kernel.
"""
import torch

from ..kernels import ops
from ..weights.loader import WeightSpec
from .base import DeferredRows, FeedForward, register_part
from .linear import linear, linear_tail


@register_part("feed_forward", "swiglu")
class SwiGLU(FeedForward):
    graph_safe = True
    accepts_deferred = True
    fuses_tail = True

    def __init__(self, name, runtime, hidden_size: int, intermediate_size: int):
        super().__init__(name, runtime)
        self.hidden_size = hidden_size
        self.intermediate_size = intermediate_size
        self.w_gate_up = None
        self.w_down = None

    def weight_specs(self):
        n, d, di = self.name, self.hidden_size, self.intermediate_size
        return {
            n + "gate_proj.weight": WeightSpec((di, d), pack=(n + "gate_up_proj.packed", 0)),
            n + "up_proj.weight": WeightSpec((di, d), pack=(n + "gate_up_proj.packed", 1)),
            n + "down_proj.weight": WeightSpec((d, di)),
        }

    def load_weights(self, tensors):
        n = self.name
        packed = tensors.get(n + "gate_up_proj.packed")      # laid out [gate; up] by the loader
        if packed is not None:
            self.w_gate_up = packed
        else:
            g, u = tensors[n + "gate_proj.weight"], tensors[n + "up_proj.weight"]
            if g.dtype != u.dtype:
                g, u = g.to(torch.float32), u.to(torch.float32)
            self.w_gate_up = torch.cat([g, u], dim=0).contiguous()
        self.w_down = tensors[n + "down_proj.weight"]

    def native_desc(self):
        from ..kernels.lib import IcSwiGLU
        ws = (self.w_gate_up, self.w_down)
        if not (self._forward_is(SwiGLU)
                and all(w is not None and w.is_cuda and w.dtype == self.runtime.dtype and w.is_contiguous() for w in ws)):
            return None
        return IcSwiGLU(self.intermediate_size, self.w_gate_up.data_ptr(), self.w_down.data_ptr())

    def forward(self, h, ctx, tail=None):
        rt = self.runtime
        if isinstance(h, DeferredRows) and h.sumsq is None:
            h = h.values                   # the whole norm is applied already: plain rows, nothing owed
        T = h.shape[0]
        act = ctx.ws.buffer("ffn_act", (T, self.intermediate_size), rt.dtype)
        owed = isinstance(h, DeferredRows)
        rows = h.values if owed else h
        few = (rt.gemm_impl == "auto" and rows.dtype == self.w_gate_up.dtype == act.dtype
               and ops.rule_gate_up_fused(rows.dtype, T, rows, self.w_gate_up, owed))
        if few:
            # few rows: the activation is the epilogue of the gate/up projection
            if isinstance(h, DeferredRows):
                ops.gemm_nt(h.values, self.w_gate_up, act, swiglu_output=True, row_factor=h.row_factor())
            else:
                ops.gemm_nt(h, self.w_gate_up, act, swiglu_output=True)
        else:
            gate_up = ctx.ws.buffer("gate_up", (T, 2 * self.intermediate_size), rt.dtype)
            linear(h, self.w_gate_up, gate_up, rt.gemm_impl, ws=ctx.ws)
            ops.swiglu(gate_up, act)
        fused = linear_tail(act, self.w_down, tail, ctx.ws, "ffn_tail", rt.gemm_impl)
        if fused is not None:
            return fused
        y = ctx.ws.buffer("ffn_out", (T, self.hidden_size), rt.dtype)
        linear(act, self.w_down, y, rt.gemm_impl, ws=ctx.ws)
        return y
