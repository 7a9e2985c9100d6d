"""Host side of the cache: pages, block tables, state slots.  No tensor is
touched here; ``storage.py`` holds the device memory these indices point into.

The reference keeps one whole-context slab per request and layer
(src/models/jiuge/jiuge_kv_cache.cpp:3-23) handed out by a Python pool
(scripts/kvcache_pool.py:18-48).  Here keys and values live in pages of
``page_size`` tokens.  Cache slots (one per entry of the model's run order that
writes a cache) with the same needs form a *group*; each group has its own
page pool and each request has one block table per group.  A group that only
needs a window of keys gives pages back once every key in them has left the
window.  Beside the pages every admitted request holds one *state slot*: an
index into fixed-size per-request state tensors.
"""
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence


class CacheError(RuntimeError):
    pass


class OutOfPages(CacheError):
    """Not enough free pages (or state slots) for what was asked."""


class PositionOverflow(CacheError):
    """A request would grow beyond the model's largest position."""


@dataclass(frozen=True)
class GroupSpec:
    """Needs of a group of cache slots.  kind 'full': every key is kept;
    'window': only the last ``window`` keys are ever read."""
    kind: str
    n_kv_heads: int
    head_dim: int
    window: Optional[int] = None
    slots: tuple = ()                   # cache slot ids (positions in the model's cache list)
    planes: int = 2                     # tensors per slot (keys and values: 2; one latent per token: 1)

    def __post_init__(self):
        if self.kind not in ("full", "window"):
            raise CacheError("group kind must be 'full' or 'window'")
        if self.kind == "window" and not (self.window and self.window > 0):
            raise CacheError("a window group needs a positive window")
        if self.planes <= 0:
            raise CacheError("a group needs at least one plane")


class PagePool:
    """Free list of page ids 0..n-1, last freed first reused."""

    def __init__(self, num_pages: int):
        if num_pages <= 0:
            raise CacheError("a page pool needs at least one page")
        self.num_pages = num_pages
        self._free: List[int] = list(range(num_pages - 1, -1, -1))   # pop() hands out 0 first
        self._is_free = [True] * num_pages

    @property
    def n_free(self) -> int:
        return len(self._free)

    def alloc(self) -> int:
        if not self._free:
            raise OutOfPages("page pool is empty")
        p = self._free.pop()
        self._is_free[p] = False
        return p

    def free(self, page: int) -> None:
        if not (0 <= page < self.num_pages):
            raise CacheError("page %r is not of this pool" % (page,))
        if self._is_free[page]:
            raise CacheError("page %d freed twice" % page)
        self._is_free[page] = True
        self._free.append(page)


class SlotPool(PagePool):
    """State slots are handed out like pages."""


@dataclass
class RequestEntry:
    state_slot: int
    length: int = 0                                  # tokens whose keys are in the cache
    tables: List[List[int]] = field(default_factory=list)   # per group: page id per logical page, -1 = given back
    first_live: List[int] = field(default_factory=list)     # per group: first logical page still held
    serial: int = 0                                  # admission number: tells two lives of one request id apart


class CacheManager:
    def __init__(self, groups: Sequence[GroupSpec], num_pages, page_size: int, max_requests: int,
                 max_positions: Optional[int] = None):
        if page_size <= 0:
            raise CacheError("page_size must be positive")
        self.groups = list(groups)
        self.page_size = page_size
        self.max_requests = max_requests
        self.max_positions = max_positions
        if isinstance(num_pages, int):
            num_pages = [num_pages] * len(self.groups)
        if len(num_pages) != len(self.groups):
            raise CacheError("one page count per group is needed")
        self.pools = [PagePool(n) for n in num_pages]
        self.slots = SlotPool(max_requests)
        self.requests: Dict[object, RequestEntry] = {}
        self._admissions = 0

    # ---- admission ------------------------------------------------------------
    def has_request(self, req_id) -> bool:
        return req_id in self.requests

    def can_admit(self) -> bool:
        return self.slots.n_free > 0

    def admit(self, req_id) -> int:
        """Give the request a state slot and empty block tables."""
        if req_id in self.requests:
            raise CacheError("request %r is already admitted" % (req_id,))
        if self.slots.n_free == 0:
            raise OutOfPages("no free state slot (max_requests = %d)" % self.max_requests)
        slot = self.slots.alloc()
        self._admissions += 1
        self.requests[req_id] = RequestEntry(
            state_slot=slot, tables=[[] for _ in self.groups], first_live=[0] * len(self.groups),
            serial=self._admissions)
        return slot

    # ---- growth ---------------------------------------------------------------
    def _pages_for(self, length: int) -> int:
        return (length + self.page_size - 1) // self.page_size

    def pages_needed(self, req_id, n_new: int) -> List[int]:
        """New pages per group that appending n_new tokens would take."""
        e = self.requests[req_id]
        want = self._pages_for(e.length + n_new)
        return [max(0, want - len(t)) for t in e.tables]

    def can_append(self, req_id, n_new: int, reserve: Optional[List[int]] = None) -> bool:
        """True when the pools hold the pages for n_new more tokens, beyond
        ``reserve`` pages per group already promised to others in this step."""
        need = self.pages_needed(req_id, n_new)
        for g, n in enumerate(need):
            if n + (reserve[g] if reserve else 0) > self.pools[g].n_free:
                return False
        return True

    def append(self, req_id, n_new: int) -> int:
        """Reserve room for n_new more tokens; returns the position of the first.
        Either every group gets its pages or nothing changes."""
        if n_new <= 0:
            raise CacheError("append needs a positive token count")
        e = self.requests[req_id]
        if self.max_positions is not None and e.length + n_new > self.max_positions:
            raise PositionOverflow("request %r would reach position %d, the model ends at %d"
                                   % (req_id, e.length + n_new, self.max_positions))
        need = self.pages_needed(req_id, n_new)
        for g, n in enumerate(need):
            if n > self.pools[g].n_free:
                raise OutOfPages("group %d needs %d pages for request %r, %d free"
                                 % (g, n, req_id, self.pools[g].n_free))
        for g, n in enumerate(need):
            for _ in range(n):
                e.tables[g].append(self.pools[g].alloc())
        start = e.length
        e.length += n_new
        return start

    def truncate(self, req_id, length: int) -> None:
        """Undo appends: the request holds ``length`` tokens again and the pages beyond them are
        given back.  Only for a step that failed before it ran (no window page of it was trimmed)."""
        e = self.requests[req_id]
        if length > e.length or length < 0:
            raise CacheError("truncate: request %r holds %d tokens, %d asked" % (req_id, e.length, length))
        keep = self._pages_for(length)
        for g, table in enumerate(e.tables):
            while len(table) > keep:
                p = table.pop()
                if p >= 0:
                    self.pools[g].free(p)
            e.first_live[g] = min(e.first_live[g], len(table))
        e.length = length

    def rename(self, old_id, new_id) -> None:
        """Hand everything ``old_id`` holds (pages, state slot, length) to ``new_id``: a new request
        takes over a finished one's cache to go on from a common prefix."""
        if new_id in self.requests:
            raise CacheError("request %r is already admitted" % (new_id,))
        e = self.requests.pop(old_id)
        self._admissions += 1
        e.serial = self._admissions               # a new life: recorded steps must not take its block table for the old one
        self.requests[new_id] = e

    def fork(self, src_id, dst_id, n_tokens: Optional[int] = None):
        """Admit ``dst_id`` with pages of its own for the first ``n_tokens`` tokens of ``src_id`` (all of
        them by default).  Returns (state slot of dst, [(group, src page, dst page), ...]): the pages whose
        contents the caller has to copy.  All or nothing: with too few pages or no slot nothing changes.
        The reference copies a cache the same way, duplicateKVCache (src/models/jiuge/jiuge_kv_cache.cpp:25-47)."""
        src = self.requests[src_id]
        n = src.length if n_tokens is None else int(n_tokens)
        if not (0 <= n <= src.length):
            raise CacheError("fork: request %r holds %d tokens, %d asked" % (src_id, src.length, n))
        if dst_id in self.requests:
            raise CacheError("request %r is already admitted" % (dst_id,))
        if self.slots.n_free == 0:
            raise OutOfPages("no free state slot (max_requests = %d)" % self.max_requests)
        n_pages = self._pages_for(n)
        live = [[j for j in range(min(n_pages, len(t))) if t[j] >= 0] for t in src.tables]
        for g, idx in enumerate(live):
            if len(idx) > self.pools[g].n_free:
                raise OutOfPages("fork needs %d pages of group %d, %d free" % (len(idx), g, self.pools[g].n_free))
        slot = self.admit(dst_id)
        dst = self.requests[dst_id]
        pairs = []
        for g, idx in enumerate(live):
            table = [-1] * n_pages                # pages the source gave back (behind a window) stay given back
            for j in idx:
                table[j] = self.pools[g].alloc()
                pairs.append((g, src.tables[g][j], table[j]))
            dst.tables[g] = table
            dst.first_live[g] = min(src.first_live[g], n_pages)
        dst.length = n
        return slot, pairs

    def trim(self, req_id) -> int:
        """Give back the pages of window groups that no later token can read.
        Call after the step that appended has been launched.  Returns the count."""
        e = self.requests[req_id]
        n = 0
        for g, spec in enumerate(self.groups):
            if spec.kind != "window":
                continue
            # the next query sits at position e.length and reads keys > e.length - window
            dead_keys = e.length - spec.window + 1            # keys < dead_keys are never read again
            dead_pages = max(0, dead_keys // self.page_size)
            for j in range(e.first_live[g], min(dead_pages, len(e.tables[g]))):
                self.pools[g].free(e.tables[g][j])
                e.tables[g][j] = -1
                n += 1
            e.first_live[g] = max(e.first_live[g], min(dead_pages, len(e.tables[g])))
        return n

    # ---- release --------------------------------------------------------------
    def release(self, req_id) -> None:
        """Give back everything the request holds."""
        e = self.requests.pop(req_id)
        for g, table in enumerate(e.tables):
            for p in reversed(table):
                if p >= 0:
                    self.pools[g].free(p)
        self.slots.free(e.state_slot)

    # ---- lookups ----------------------------------------------------------------
    def length(self, req_id) -> int:
        return self.requests[req_id].length

    def state_slot(self, req_id) -> int:
        return self.requests[req_id].state_slot

    def block_table(self, req_id, group: int) -> List[int]:
        return self.requests[req_id].tables[group]

    def slot_of(self, req_id, group: int, position: int) -> int:
        """Physical token slot (page * page_size + offset) of a position."""
        page = self.requests[req_id].tables[group][position // self.page_size]
        if page < 0:
            raise CacheError("position %d of request %r lies in a page that was given back" % (position, req_id))
        return page * self.page_size + position % self.page_size

    def free_pages(self, group: int = 0) -> int:
        return self.pools[group].n_free

    def check_invariants(self) -> None:
        """Every page is either free or held by exactly one request."""
        for g, pool in enumerate(self.pools):
            held = []
            for e in self.requests.values():
                held.extend(p for p in e.tables[g] if p >= 0)
            if len(held) != len(set(held)):
                raise CacheError("group %d: a page is held twice" % g)
            free = set(pool._free)
            if len(free) != len(pool._free):
                raise CacheError("group %d: a page is on the free list twice" % g)
            if free & set(held):
                raise CacheError("group %d: a held page is on the free list" % g)
            if len(free) + len(held) != pool.num_pages:
                raise CacheError("group %d: %d pages lost" % (g, pool.num_pages - len(free) - len(held)))
        slots = [e.state_slot for e in self.requests.values()]
        if len(slots) != len(set(slots)) or len(slots) + self.slots.n_free != self.max_requests:
            raise CacheError("state slots lost or held twice")
