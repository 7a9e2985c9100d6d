"""What one step hands to the parts: the batch as flat arrays, the cache views
and the workspace.

A batch is a list of (request, its next tokens).  Tokens are concatenated in
entry order, as the reference does (src/models/jiuge/jiuge.cpp:147-154):
``positions[t] = req_pos[r] + i``.  All integer arrays of a step are packed
into one pinned host buffer and reach the device in one copy.
"""
from dataclasses import dataclass
from typing import Dict, List, Optional

import torch


class Workspace:
    """Named scratch buffers that grow to the largest size asked for and are then
    reused, so steps of a steady shape allocate nothing and pointers stay put."""

    def __init__(self, device):
        self.device = device
        self._bufs: Dict[tuple, torch.Tensor] = {}
        self._views: Dict[tuple, tuple] = {}     # (name, dtype) -> (shape, view): the view handed out last
        self.frozen = False                      # True: buffers may not be regrown (recorded launches hold their addresses)

    def buffer(self, name: str, shape, dtype) -> torch.Tensor:
        key = (name, dtype)
        shape = tuple(shape)
        last = self._views.get(key)
        if last is not None and last[0] == shape:       # the usual case: the same shape as last time
            return last[1]
        n = 1
        for s in shape:
            n *= int(s)
        buf = self._bufs.get(key)
        if buf is None or buf.numel() < n:
            if self.frozen:
                raise RuntimeError("workspace buffer %r would have to grow from %d to %d elements, but recorded "
                                   "steps hold its address" % (name, 0 if buf is None else buf.numel(), n))
            buf = torch.empty(max(n, 1), dtype=dtype, device=self.device)
            self._bufs[key] = buf
        view = buf[:n].view(*shape)
        self._views[key] = (shape, view)
        return view

    def zeroed(self, name: str, shape, dtype) -> torch.Tensor:
        """A buffer of a fixed shape that is zero when it is first handed out and is the caller's to keep so (arrival
        counters that every launch leaves at zero).  It is never regrown, so what it holds is never lost."""
        key = (name, dtype)
        shape = tuple(shape)
        buf = self._bufs.get(key)
        if buf is None:
            if self.frozen:
                raise RuntimeError("workspace buffer %r would have to be made, but recorded steps hold the workspace" % name)
            buf = torch.zeros(shape, dtype=dtype, device=self.device)
            self._bufs[key] = buf
        elif tuple(buf.shape) != shape:
            raise RuntimeError("workspace buffer %r has a fixed shape %s, asked for %s" % (name, tuple(buf.shape), shape))
        return buf

    def bytes(self) -> int:
        return sum(b.numel() * b.element_size() for b in self._bufs.values())


@dataclass
class LayerCacheView:
    """What a mixer sees of its cache slot in this step: the planes of its paged memory (if it asked for
    any) with the step's token slots and block tables, and its fixed-size state (if it asked for one)."""
    k: Optional[torch.Tensor] = None             # plane 0 [pages, kv_heads, page_size, head_dim]
    v: Optional[torch.Tensor] = None             # plane 1 (None for a slot with one plane)
    slots: Optional[torch.Tensor] = None         # int32 [T]: token slot of each new token in this group
    block_tables: Optional[torch.Tensor] = None  # int32 [R, max_blocks]
    state: Optional[torch.Tensor] = None         # [max_requests, ...] fixed-size state of this slot
    writes: bool = True
    planes: tuple = ()                           # every plane of the slot, in order (k and v are the first two)

    @classmethod
    def of_planes(cls, planes, slots, block_tables, state=None) -> "LayerCacheView":
        return cls(k=planes[0], v=planes[1] if len(planes) > 1 else None, slots=slots, block_tables=block_tables,
                   state=state, planes=tuple(planes))


class StepContext:
    """Flat description of a step's batch.  Built by ``Engine``; read by parts."""

    def __init__(self):
        self.T = 0                       # tokens in the step
        self.R = 0                       # requests in the step
        self.page_size = 0
        self.ws: Workspace = None
        # device arrays
        self.tokens = None               # int32 [T]
        self.positions = None            # int32 [T]
        self.token_req = None            # int32 [T]  batch row of each token
        self.state_slots = None          # int32 [R]  state slot of each request
        self.want_rows = None            # int32 [W]  token rows whose logits are wanted
        self.n_want = 0
        self.want_rows_identity = False  # every row's logits are wanted, in order
        # listed when some part of the model asks for them (Part.portion_tile_rows):
        self.decode_rows = None          # int32 [n_decode_rows] rows that are a request's single token
        self.n_decode_rows = 0
        self.decode_rows_identity = False
        self.prefill_tiles = None        # int32 [n_tiles, 4] (batch row, first token row, rows, first position)
        self.n_prefill_tiles = 0
        # host copies
        self.req_start: List[int] = []   # first token row of each request (R + 1 entries)
        self.req_pos: List[int] = []     # position of each request's first new token
        self.req_len: List[int] = []
        self.req_ids: List[object] = []
        self.host_state_slots: List[int] = []
        self.max_position = 0            # largest position in the step
        self.max_context = 0             # most keys any single-token row sees
        self.cu_count = 256              # compute units of the device, for the parts' launch heuristics
        self.fixed_decode_splits: Optional[int] = None   # a recorded step's fixed way of splitting single-token rows' keys
        self.memo: Dict[str, object] = {}  # scratch of the parts for this step (what several layers would work out alike)
        self.group_views = []            # per cache group: (slots int32 [T], block tables int32 [R, max_blocks])
        self._views: Dict[int, LayerCacheView] = {}

    def cache_view(self, entry) -> LayerCacheView:
        v = self._views[entry.cache]
        if v.writes != entry.writes_cache:
            v = LayerCacheView(v.k, v.v, v.slots, v.block_tables, v.state, entry.writes_cache, v.planes)
        return v
