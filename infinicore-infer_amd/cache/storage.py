"""Device memory of the cache: the page planes of each group and the
per-request state tensors.

Layout of one plane of a cache slot (one attention layer's keys or values):
``[num_pages, n_kv_heads, page_size, head_dim]``: the keys of one head inside a
page are one contiguous run, which is what the attention kernels stream.
A group holds ``[n_slots, planes, num_pages, n_kv_heads, page_size, head_dim]``;
attention has two planes (K, V), a mixer that caches one vector per token has one.
"""
from typing import Dict, List, Sequence, Tuple

import torch

from .manager import GroupSpec


class CacheStorage:
    def __init__(self, groups: Sequence[GroupSpec], num_pages: Sequence[int], page_size: int,
                 dtype: torch.dtype, device):
        self.page_size = page_size
        self.dtype = dtype
        self.device = device
        self.group_planes: List[torch.Tensor] = []
        self._slot_index: Dict[int, Tuple[int, int]] = {}      # cache slot -> (group, index in group)
        for g, spec in enumerate(groups):
            planes = torch.empty((len(spec.slots), spec.planes, num_pages[g], spec.n_kv_heads, page_size, spec.head_dim),
                                 dtype=dtype, device=device)
            self.group_planes.append(planes)
            for i, s in enumerate(spec.slots):
                self._slot_index[s] = (g, i)
        self.state: Dict[int, torch.Tensor] = {}               # cache slot -> [max_requests, ...]
        self._kv_views: Dict[int, tuple] = {}
        self._copy_idx = None                                  # (pinned, device) page ids of copy_pages, kept between calls

    def add_state(self, slot: int, max_requests: int, shape, dtype) -> torch.Tensor:
        t = torch.zeros((max_requests,) + tuple(shape), dtype=dtype, device=self.device)
        self.state[slot] = t
        return t

    def group_of(self, slot: int) -> int:
        return self._slot_index[slot][0]

    def planes(self, slot: int) -> tuple:
        """The planes of a cache slot, each [num_pages, n_kv_heads, page_size, head_dim] (views made
        once: the planes never move)."""
        views = self._kv_views.get(slot)
        if views is None:
            g, i = self._slot_index[slot]
            views = self._kv_views[slot] = tuple(self.group_planes[g][i, j] for j in range(self.group_planes[g].shape[1]))
        return views

    def kv(self, slot: int):
        """(K plane, V plane) of a cache slot with two planes."""
        views = self.planes(slot)
        if len(views) != 2:
            raise ValueError("cache slot %d has %d planes, not keys and values" % (slot, len(views)))
        return views

    def copy_pages(self, group: int, src_pages: Sequence[int], dst_pages: Sequence[int]) -> None:
        """Copy whole pages inside a group: every cache slot of the group, every plane."""
        if not src_pages:
            return
        from ..kernels import ops
        planes = self.group_planes[group]
        n = len(src_pages)
        # page ids through a pinned buffer into device memory that is kept (grown to the largest copy asked for)
        if self._copy_idx is None or self._copy_idx[0].shape[1] < n:
            cap = max(n, 64)
            self._copy_idx = (torch.empty(2, cap, dtype=torch.int32, pin_memory=True),
                              torch.empty(2, cap, dtype=torch.int32, device=self.device))
        host, dev = self._copy_idx
        torch.cuda.current_stream().synchronize()          # the copy before has read the pinned buffer
        host[0, :n] = torch.as_tensor(list(src_pages), dtype=torch.int32)
        host[1, :n] = torch.as_tensor(list(dst_pages), dtype=torch.int32)
        dev.copy_(host, non_blocking=True)
        ops.copy_pages(planes, dev[0, :n], dev[1, :n])

    def copy_state(self, src_slot: int, dst_slot: int) -> None:
        for t in self.state.values():
            t[dst_slot].copy_(t[src_slot])

    def zero_state(self, state_slot: int) -> None:
        for t in self.state.values():
            t[state_slot].zero_()

    def bytes(self) -> int:
        n = sum(p.numel() * p.element_size() for p in self.group_planes)
        return n + sum(t.numel() * t.element_size() for t in self.state.values())
