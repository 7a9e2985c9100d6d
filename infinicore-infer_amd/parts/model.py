"""The layered model: an embedding, layers run in the order a list gives, a
final norm and a head.  Built from a ``ModelSpec``; knows no architecture.

Forward of one step (src/models/jiuge/jiuge.cpp:164-168,195-258,261-278 is the
reference's): gather embeddings into the float32 residual stream, run the
schedule, settle the last residual add, then normalise and project only the
rows whose logits are wanted.
"""
from typing import Dict, List

import torch

from ..config.spec import ModelSpec
from ..kernels import ops
from ..weights.loader import WeightSpec, load_weights
from .base import CacheNeed, DeferredRows, Runtime, build_part


class DecoderModel:
    def __init__(self, spec: ModelSpec, runtime: Runtime):
        self.spec = spec
        self.runtime = runtime
        memo = {}
        self.embedding = build_part("embedding", spec.embedding, runtime, memo)
        self.layers = []
        for ls in spec.layers:
            opt = lambda category, spec: None if spec is None else build_part(category, spec, runtime, memo)
            mixer = opt("mixer", ls.mixer)
            ffn = opt("feed_forward", ls.feed_forward)
            n1 = opt("norm", ls.mixer_norm)
            n2 = opt("norm", ls.feed_forward_norm)
            from .base import _REGISTRY
            try:
                block_cls = _REGISTRY["block"][ls.block.kind]
            except KeyError:
                raise KeyError("no block part of kind %r" % ls.block.kind)
            self.layers.append(block_cls(ls.block.name, runtime, mixer=mixer, mixer_norm=n1, feed_forward=ffn,
                                         feed_forward_norm=n2, **ls.block.params))
        self.final_norm = build_part("norm", spec.final_norm, runtime, memo)
        self.head = build_part("head", spec.head, runtime, memo)
        self.schedule = list(spec.schedule)
        for e in self.schedule:
            if not (0 <= e.layer < len(self.layers)):
                raise ValueError("run order names layer %d, the model has %d" % (e.layer, len(self.layers)))
        writers = {}
        for e in self.schedule:
            if e.writes_cache:
                if e.cache in writers:
                    raise ValueError("cache slot %d is written by two entries of the run order" % e.cache)
                writers[e.cache] = e.layer
        for e in self.schedule:
            if not e.writes_cache and e.cache not in writers:
                raise ValueError("cache slot %d is read but never written" % e.cache)
        self._writers = writers
        # an entry that reads another entry's cache must fit what the writer keeps: the same heads and
        # head size, and no more keys than the writer's window holds (pages behind a window are given
        # back and their block-table entries are reused)
        for e in self.schedule:
            if e.writes_cache:
                continue
            wn = self._cache_need_of(writers[e.cache])
            rn = self._cache_need_of(e.layer)
            if not (wn.paged and rn.paged):
                continue
            if (rn.planes, rn.n_kv_heads, rn.head_dim) != (wn.planes, wn.n_kv_heads, wn.head_dim):
                raise ValueError("layer %d reads cache slot %d as %d planes with %d kv heads of %d, its writer (layer %d) "
                                 "keeps %d planes with %d of %d" % (e.layer, e.cache, rn.planes, rn.n_kv_heads, rn.head_dim,
                                                                    writers[e.cache], wn.planes, wn.n_kv_heads, wn.head_dim))
            if wn.window and (not rn.window or rn.window > wn.window):
                raise ValueError("layer %d reads cache slot %d over %s keys, its writer (layer %d) keeps a window of %d"
                                 % (e.layer, e.cache, rn.window or "all", writers[e.cache], wn.window))

    # ---- parts and weights ---------------------------------------------------------
    def all_parts(self):
        seen, out = set(), []

        def walk(p):
            if id(p) in seen:
                return
            seen.add(id(p))
            out.append(p)
            for s in p.sub_parts():
                walk(s)
        walk(self.embedding)
        for l in self.layers:
            walk(l)
        walk(self.final_norm)
        walk(self.head)
        return out

    def weight_specs(self) -> Dict[str, WeightSpec]:
        specs: Dict[str, WeightSpec] = {}
        for p in self.all_parts():
            for name, s in p.weight_specs().items():
                if name in specs and specs[name] != s:
                    raise ValueError("tensor %s is wanted with two different specs" % name)
                specs[name] = s
        return specs

    def load_weights(self, tensors: Dict[str, torch.Tensor]) -> None:
        for p in self.all_parts():
            p.load_weights(tensors)

    def load_from_dir(self, model_dir: str) -> None:
        tensors = load_weights(model_dir, self.weight_specs(), self.runtime.dtype, self.runtime.device)
        self.load_weights(tensors)

    # ---- cache needs ------------------------------------------------------------------
    def _cache_need_of(self, layer: int) -> CacheNeed:
        mixer = self.layers[layer].mixer
        return CacheNeed() if mixer is None else mixer.cache_need()       # a layer without a mixer keeps nothing

    def cache_needs(self) -> List[CacheNeed]:
        """One need per cache slot, in slot order."""
        n = self.spec.num_cache_slots()
        needs = [CacheNeed() for _ in range(n)]
        for slot, layer in self._writers.items():
            needs[slot] = self._cache_need_of(layer)
        return needs

    def weight_bytes(self) -> int:
        seen, total = set(), 0
        for p in self.all_parts():
            for v in vars(p).values():
                if isinstance(v, torch.Tensor) and v.data_ptr() not in seen:
                    seen.add(v.data_ptr())
                    total += v.numel() * v.element_size()
        return total

    # ---- one step ------------------------------------------------------------------------
    def forward(self, ctx):
        """Runs ctx.T tokens; returns float32 logits [len(ctx.want_rows), vocab] or None."""
        T = ctx.T
        x = ctx.ws.buffer("residual", (T, self.spec.hidden_size), torch.float32)
        self.embedding.forward(ctx.tokens, x)
        pending = None
        last = len(self.schedule) - 1
        for i, e in enumerate(self.schedule):
            block = self.layers[e.layer]
            if not block.fuses_successor:
                if isinstance(pending, DeferredRows):
                    raise RuntimeError("block %s was handed half-normed rows it did not ask for" % block.name)
                pending = block.forward(x, pending, ctx, ctx.cache_view(e))
                continue
            # the norm that runs next, if whoever applies it can take its rows half done
            if i < last:
                successor = self.layers[self.schedule[i + 1].layer].entry_norm()
            elif ctx.want_rows_identity and getattr(self.head, "accepts_deferred", False):
                successor = self.head.deferred_norm(self.final_norm)
            else:
                successor = None
            pending = block.forward(x, pending, ctx, ctx.cache_view(e), successor=successor)
        if ctx.n_want == 0:
            return None
        if isinstance(pending, DeferredRows):
            return self.head.forward(pending, ctx.want_rows, self.final_norm, ctx)
        if pending is not None:
            ops.residual_add(x, pending[0], pending[1])
        return self.head.forward(x, ctx.want_rows, self.final_norm, ctx)


def build_model(spec: ModelSpec, runtime: Runtime) -> DecoderModel:
    return DecoderModel(spec, runtime)
