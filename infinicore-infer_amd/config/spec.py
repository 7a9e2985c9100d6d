"""Architecture-neutral description of a model: what the configuration layer
hands to the part builders.

A model is data: an embedding, a list of layers (each naming its mixer,
feed-forward, two norms and the block arrangement that joins them), the order
in which layers run, a final norm and an output head.  Every size and constant
is a parameter in a ``PartSpec``; no part looks at a model-level configuration.
"""
from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional


@dataclass(frozen=True)
class PartSpec:
    """One part: ``kind`` selects the class in the part registry, ``name`` is the
    prefix of its tensors in the weight file, ``params`` are its constructor
    arguments (sizes, constants, nested PartSpecs)."""
    kind: str
    name: str = ""
    params: Dict[str, Any] = field(default_factory=dict)


@dataclass(frozen=True)
class LayerSpec:
    """A layer = a block arrangement over the parts it names.  Which parts a layer must have is the
    block kind's question: the pre-norm residual block wants a mixer with its norm and takes a
    feed-forward with its norm or none (a stack of mixers alone); another arrangement (one norm
    shared by mixer and feed-forward, a feed-forward alone) names what it uses and leaves the rest None."""
    block: PartSpec
    mixer: Optional[PartSpec] = None
    mixer_norm: Optional[PartSpec] = None
    feed_forward: Optional[PartSpec] = None
    feed_forward_norm: Optional[PartSpec] = None


@dataclass(frozen=True)
class ExecEntry:
    """One entry of the run order.

    ``layer``   index into ``ModelSpec.layers`` (a layer may appear twice: its
                weights are then shared).
    ``cache``   index of the cache slot this entry's mixer uses.  By default
                every entry has a slot of its own.
    ``writes_cache``  False when the entry only reads a slot that an earlier
                entry wrote (a layer reading another layer's cache).
    """
    layer: int
    cache: int
    writes_cache: bool = True


@dataclass(frozen=True)
class ModelSpec:
    architecture: str
    vocab_size: int
    hidden_size: int
    max_positions: int
    embedding: PartSpec
    layers: List[LayerSpec]
    schedule: List[ExecEntry]
    final_norm: PartSpec
    head: PartSpec
    eos_token_ids: List[int] = field(default_factory=list)
    bos_token_id: Optional[int] = None

    def num_cache_slots(self) -> int:
        return 1 + max((e.cache for e in self.schedule), default=-1)


def default_schedule(num_layers: int) -> List[ExecEntry]:
    """Layers 0..L-1 once each, each with its own cache slot."""
    return [ExecEntry(layer=i, cache=i, writes_cache=True) for i in range(num_layers)]
