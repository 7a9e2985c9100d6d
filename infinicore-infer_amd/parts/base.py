"""Interfaces of the parts a layer is put together from, and their registry.

Categories: ``mixer`` (attention here), ``feed_forward``, ``norm``,
``position_encoding``, ``block`` (the arrangement of the others in a layer),
``embedding`` and ``head``.  A part is built from a ``PartSpec``: its class is
looked up by ``(category, kind)`` and called as ``cls(name, runtime, **params)``.
A part sees its own parameters, the step's batch description and the cache
view it is handed; it never sees the model or its configuration.
"""
from dataclasses import dataclass
from typing import Callable, Dict, Optional, Tuple

import torch

from ..config.spec import PartSpec
from ..weights.loader import WeightSpec

CATEGORIES = ("mixer", "feed_forward", "norm", "position_encoding", "block", "embedding", "head")
_REGISTRY: Dict[str, Dict[str, type]] = {c: {} for c in CATEGORIES}


@dataclass(frozen=True)
class Runtime:
    """What every part needs to know about where and how it computes."""
    dtype: torch.dtype                 # compute dtype of activations and cache: bfloat16 or float32
    device: object                     # torch device of weights and buffers
    attention_impl: str = "auto"       # "auto": tiled kernels where they apply; "generic": the general kernel only
    gemm_impl: str = "auto"            # "auto": own kernel for few rows; "library": always the library GEMM


@dataclass(frozen=True)
class CacheNeed:
    """What a mixer needs from the cache manager.
    kind 'kv': paged memory, ``planes`` tensors per cache slot that hold ``n_kv_heads`` rows of
    ``head_dim`` values for every token (keys and values of attention: 2 planes; one latent vector
    per token: planes = 1, n_kv_heads = 1, head_dim = its width), all tokens or a window of them;
    kind 'state': a fixed-size tensor of ``state_shape`` per request;
    kind 'kv+state': both, for a mixer that walks a paged cache and carries a running state as well;
    kind 'none': nothing."""
    kind: str = "none"
    n_kv_heads: int = 0
    head_dim: int = 0
    window: Optional[int] = None
    state_shape: Tuple[int, ...] = ()
    state_dtype: torch.dtype = torch.float32
    planes: int = 2

    def __post_init__(self):
        if self.kind not in ("none", "kv", "state", "kv+state"):
            raise ValueError("cache need of kind %r (have none, kv, state, kv+state)" % (self.kind,))
        if self.paged and (self.n_kv_heads <= 0 or self.head_dim <= 0 or self.planes <= 0):
            raise ValueError("a paged cache need names planes, rows per token and their width (got %d, %d, %d)"
                             % (self.planes, self.n_kv_heads, self.head_dim))
        if self.has_state and not self.state_shape:
            raise ValueError("a state need names the state's shape")

    @property
    def paged(self) -> bool:
        return self.kind in ("kv", "kv+state")

    @property
    def has_state(self) -> bool:
        return self.kind in ("state", "kv+state")


@dataclass
class DeferredRows:
    """Rows whose norm is half done.  ``values[r]`` is x[r] * w (the norm's weight is applied, its
    row factor is not); ``sumsq[b, r]`` are sums of x[r]^2 over column blocks b.  The true row is
    values[r] * rsqrt(sumsq[:, r].sum() / width + eps).  The row factor commutes with a projection,
    so a part that takes such rows (``accepts_deferred``) applies it to its first product's result.
    ``sumsq`` None: the producer has applied the whole norm already and ``values`` are the normed rows
    (nothing is owed); consumers then treat them as a plain tensor."""
    values: torch.Tensor
    sumsq: Optional[torch.Tensor]      # float32 [n_parts, 16], or None
    width: int
    eps: float

    @property
    def shape(self):
        return self.values.shape

    @property
    def dtype(self):
        return self.values.dtype

    def row_factor(self):
        return None if self.sumsq is None else (self.sumsq, self.width, self.eps)

    def materialize(self):
        """The normed rows as a plain tensor (slow path for parts of a product that cannot take factors)."""
        if self.sumsq is None:
            return self.values
        T = self.values.shape[0]
        f = torch.rsqrt(self.sumsq.sum(0)[:T, None] / self.width + self.eps)
        return (self.values.to(torch.float32) * f).to(self.values.dtype)


@dataclass
class ResidualTail:
    """What a block asks of a part's LAST projection (a part with ``fuses_tail``): add the part's
    output y to the float32 residual stream, x += alpha * y, and hand back the input of the norm
    that follows (weight, eps) as ``DeferredRows``.  A part that cannot do it for this step returns
    its plain output and the block does the add and the norm itself."""
    x: torch.Tensor
    alpha: float
    weight: torch.Tensor
    eps: float


def register_part(category: str, kind: str) -> Callable:
    if category not in _REGISTRY:
        raise KeyError("unknown part category %r (have %s)" % (category, ", ".join(CATEGORIES)))

    def _do(cls):
        _REGISTRY[category][kind] = cls
        return cls
    return _do


def registered_parts(category: str):
    return sorted(_REGISTRY[category])


def build_part(category: str, spec: PartSpec, runtime: Runtime, memo: Optional[dict] = None):
    """Instantiate the part a spec names.  ``memo`` (id(spec) -> part) lets
    several layers share one instance of the same spec object."""
    if memo is not None and id(spec) in memo:
        return memo[id(spec)]
    try:
        cls = _REGISTRY[category][spec.kind]
    except KeyError:
        raise KeyError("no %s part of kind %r; registered: %s"
                       % (category, spec.kind, ", ".join(registered_parts(category))))
    part = cls(spec.name, runtime, **spec.params)
    if memo is not None:
        memo[id(spec)] = part
    return part


class Part:
    """Base of all parts."""
    category = ""
    # True when forward() launches the same kernels with the same arguments for every step of
    # a given batch shape and reads the step's integers only from device arrays (never from the
    # context's host lists): such a step can be recorded once and replayed.
    graph_safe = False

    def __init__(self, name: str, runtime: Runtime):
        self.name = name
        self.runtime = runtime

    def weight_specs(self) -> Dict[str, WeightSpec]:
        """Full tensor name -> what is expected of it."""
        return {}

    def load_weights(self, tensors: Dict[str, torch.Tensor]) -> None:
        """Take this part's tensors (keys as in weight_specs) from ``tensors``."""

    def sub_parts(self):
        return ()

    def native_desc(self):
        """What the native step function needs to run this part without Python: a description struct
        of the kernel library's C interface (sizes, constants, weight addresses), or None when the
        part has no native counterpart (then the whole model is stepped from Python).  A part that
        overrides ``forward`` of a built-in part must not inherit its description."""
        return None

    def _forward_is(self, cls) -> bool:
        """True when this object's forward is ``cls``'s own (no subclass changed what a step does)."""
        return type(self).forward is cls.forward

    def portion_tile_rows(self):
        """Rows per tile when this part wants the step's batch listed as tiles of prompt portions and
        rows of single tokens (``StepContext.prefill_tiles`` and ``decode_rows``), else None.  Parts of
        one model that ask must ask for the same tile height."""
        return None

    def position_limit(self):
        """Positions this part can take (a table's length), or None when it has no limit.  The
        engine refuses a step that would go beyond the smallest limit before it changes anything."""
        return None


class Norm(Part):
    category = "norm"

    def forward(self, x, out, rows=None, out_scale: float = 1.0):
        """out[r] = norm(x[rows[r] or r]) * out_scale; x is the float32 residual stream."""
        raise NotImplementedError

    def forward_add(self, x, y, alpha: float, out):
        """x += alpha * y, then out = norm(x).  Parts without a fused kernel inherit this."""
        from ..kernels import ops
        ops.residual_add(x, y, alpha)
        return self.forward(x, out)

    def deferred(self):
        """(weight, eps) when the norm is y = x * rsqrt(mean(x^2) + eps) * weight, so that it can be
        split over the products before and after it (``DeferredRows``); None otherwise."""
        return None


class PositionEncoding(Part):
    category = "position_encoding"

    def rotate_and_store(self, qkv, ctx, cache, n_heads: int, n_kv_heads: int, head_dim: int):
        """Encode positions into the q (and k) heads of qkv[T, H] in place and,
        when n_kv_heads > 0, write k and v into ``cache`` at the step's slots."""
        raise NotImplementedError

    def project_rotate_store(self, h, w_qkv, qkv, ctx, cache, n_heads: int, n_kv_heads: int, head_dim: int) -> bool:
        """Optional shortcut: compute qkv = h w_qkv^T AND do what rotate_and_store does, in one
        kernel.  Returns False (nothing done) when the part has no such kernel for this case."""
        return False


class Mixer(Part):
    category = "mixer"
    accepts_deferred = False     # forward() takes DeferredRows as h
    fuses_tail = False           # forward() takes tail=ResidualTail and may return DeferredRows

    def cache_need(self) -> CacheNeed:
        return CacheNeed()

    def forward(self, h, ctx, cache):
        """h: [T, hidden] normed input in the compute dtype; returns [T, hidden]."""
        raise NotImplementedError


class FeedForward(Part):
    category = "feed_forward"
    accepts_deferred = False
    fuses_tail = False

    def forward(self, h, ctx):
        raise NotImplementedError


class Block(Part):
    """Arrangement of a mixer and a feed-forward around the residual stream.
    ``pending`` is a branch output whose residual add is still owed, as
    ``(y, alpha)``; a block may hand its last add on to the next block's norm."""
    category = "block"

    def __init__(self, name, runtime, mixer=None, mixer_norm=None, feed_forward=None, feed_forward_norm=None):
        """Any of the four may be None: a layer names the parts its arrangement uses (a subclass says which it needs)."""
        super().__init__(name, runtime)
        self.mixer = mixer
        self.mixer_norm = mixer_norm
        self.feed_forward = feed_forward
        self.feed_forward_norm = feed_forward_norm

    def sub_parts(self):
        return tuple(p for p in (self.mixer, self.mixer_norm, self.feed_forward, self.feed_forward_norm) if p is not None)

    # A block with ``fuses_successor`` is called as forward(x, pending, ctx, cache, successor=norm):
    # ``successor`` is the norm that whoever runs next applies first (None: unknown or not splittable),
    # and the block may return DeferredRows for it instead of a pending add.  ``entry_norm()`` names
    # the norm a block applies to the incoming stream when it takes DeferredRows as ``pending``.
    fuses_successor = False

    def entry_norm(self):
        return None

    def forward(self, x, pending, ctx, cache):
        raise NotImplementedError
