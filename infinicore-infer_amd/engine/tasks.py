"""Request state, in the reference's manner (scripts/infer_task.py).

``InferTask(id, tokens, max_tokens, temperature, topk, topp, end_tokens)``
carries the tokens still to be fed, the position they start at and the
sampling options; ``next(out_token)`` advances it and sets ``finish_reason``
to "stop" (an end token) or "length" (position reached ``max_tokens``), exactly
as scripts/infer_task.py:27-36 does.  ``KVCache`` is the handle a task binds:
here a request id of the engine's paged cache instead of a whole-context slab
(scripts/infer_task.py:39-59).
"""
import itertools
from typing import List, Optional, Sequence

from ..sampling.params import SamplingParams

_next_handle = itertools.count()


class KVCache:
    """A request's place in the engine's cache.  Pages are taken as tokens arrive
    and given back by ``drop``."""

    def __init__(self, model):
        self._engine = model.engine if hasattr(model, "engine") else model
        self.handle = "kv%d" % next(_next_handle)
        self.tokens: List[int] = []            # token ids stored so far (scripts/infer_task.py:42)

    def data(self):
        return self.handle

    def drop(self, model=None):
        self._engine.free(self.handle)
        self.tokens = []

    def update_tokens(self, tokens: Sequence[int], pos: int):
        del self.tokens[pos:]
        self.tokens.extend(int(t) for t in tokens)


class InferTask:
    def __init__(self, id, tokens, max_tokens, temperature=1.0, topk=1, topp=1.0, end_tokens=(),
                 seed: int = 0, max_new_tokens: Optional[int] = None):
        SamplingParams(temperature, topk, topp, seed)      # refuses a negative temperature, topp outside [0, 1], ...
        self.id = id
        self.finish_reason = None
        self.tokens = list(tokens)             # tokens to feed in the next step
        self.max_tokens = max_tokens           # limit on the absolute position (scripts/infer_task.py:33)
        self.temperature = temperature
        self.topk = topk
        self.topp = topp
        self.end_tokens = list(end_tokens)
        self.seed = seed
        self.max_new_tokens = max_new_tokens
        self._kv_cache = None
        self.pos = 0
        self.prompt = list(tokens)
        self.generated: List[int] = []

    def bind_kvcache(self, kv_cache, pos=0):
        self._kv_cache = kv_cache
        self.pos = pos
        self.tokens = self.tokens[pos:]

    def release_kvcache(self):
        cache = self._kv_cache
        self._kv_cache = None
        return cache

    def kvcache(self):
        return self._kv_cache

    def next(self, out_token):
        if self._kv_cache is not None:
            self._kv_cache.update_tokens(self.tokens, self.pos)
        self.pos += len(self.tokens)
        if out_token is not None:
            self.generated.append(int(out_token))
        if out_token is None or out_token in self.end_tokens:
            self.finish_reason = "stop"
        elif self.pos >= self.max_tokens:
            self.finish_reason = "length"
        elif self.max_new_tokens is not None and len(self.generated) >= self.max_new_tokens:
            self.finish_reason = "length"
        else:
            self.tokens = [int(out_token)]
