"""The step function: a batch of (request, its next tokens) runs as one batch
from the cache and returns the logits at the wanted places.

The reference's step is inferBatch / forwardBatch
(include/infinicore_infer/models/jiuge.h:89-110, src/models/jiuge/jiuge.cpp:114-298):
tokens of all requests concatenated, req_lens, req_pos and one cache handle per
request.  Here the cache handle is a request id known to the cache manager;
portions of prompts and single decoded tokens may be mixed and cut anywhere.
"""
from dataclasses import dataclass, field
from collections import OrderedDict
from typing import Dict, List, Optional, Sequence

import numpy as np
import torch

from ..cache import CacheManager, CacheStorage, GroupSpec, OutOfPages, PositionOverflow
from ..config import config_from_dir
from ..kernels import ops
from ..parts import Runtime, build_model
from .context import LayerCacheView, StepContext, Workspace


@dataclass
class StepEntry:
    """One request's share of a step: its next tokens and the places among them
    whose logits are wanted (indices into ``tokens``; may be empty)."""
    req_id: object
    tokens: Sequence[int]
    want: Sequence[int] = field(default_factory=list)


def _align4(n: int) -> int:
    return (n + 3) & ~3


def _context_bucket(n_keys: int) -> int:
    """The key count a step's key split is chosen for: the kernel library's rounding (one rule for steps issued from
    here, for recorded ones and for the native step function, so that they split alike)."""
    return ops.rule_context_bucket(n_keys)


class _PinnedRing:
    """A few pinned host buffers used in turn, each guarded by an event, so a
    buffer is not rewritten while its copy to the device may still run."""

    def __init__(self, n: int = 4):
        self.bufs = [None] * n
        self.events = [None] * n
        self.i = 0

    def get(self, numel: int) -> torch.Tensor:
        self.i = (self.i + 1) % len(self.bufs)
        if self.events[self.i] is not None:
            self.events[self.i].synchronize()
        b = self.bufs[self.i]
        if b is None or b.numel() < numel:
            b = torch.empty(max(numel, 1024), dtype=torch.int32, pin_memory=True)
            self.bufs[self.i] = b
        return b

    def mark(self):
        ev = self.events[self.i]
        if ev is None:
            ev = torch.cuda.Event()
            self.events[self.i] = ev
        ev.record()


class Engine:
    def __init__(self, model, max_tokens: int, page_size: int = 16, max_requests: int = 64,
                 num_pages: Optional[int] = None, use_graphs: bool = True, graph_max_batch: int = 64,
                 use_native: bool = True, max_graphs: int = 32, graph_after: int = 2):
        """``max_tokens``: the most tokens live requests hold at any time, each
        request's count rounded up to whole pages; every group's pool is sized for it.
        ``use_native``: let one native call issue a step's kernels when every part of the model
        has a native description (otherwise, and for other models, the parts' Python forward runs).
        ``max_graphs``: recorded decode steps kept at a time (the least recently used one goes first).
        ``graph_after``: a decode step's shape (batch size, key-count bucket) is recorded at its n-th appearance
        and runs eagerly before that (1: at once)."""
        self.model = model
        self.runtime: Runtime = model.runtime
        self.device = torch.device(self.runtime.device)
        if self.device.type != "cuda":
            raise RuntimeError("the engine runs on the GPU only (device %s given); there is no CPU path"
                               % self.device)
        ops.get_lib()                       # fail now, loudly, if the kernels are missing
        self.page_size = int(page_size)
        self.max_requests = int(max_requests)
        if num_pages is None:
            num_pages = (int(max_tokens) + self.page_size - 1) // self.page_size
        self.num_pages = int(num_pages)

        # ---- cache groups from the mixers' needs -------------------------------------
        needs = model.cache_needs()
        keyed: Dict[tuple, List[int]] = {}
        for slot, need in enumerate(needs):
            if need.paged:
                keyed.setdefault((need.planes, need.n_kv_heads, need.head_dim, need.window), []).append(slot)
        self.groups: List[GroupSpec] = [
            GroupSpec("window" if w else "full", nkv, dh, w, tuple(slots), planes)
            for (planes, nkv, dh, w), slots in keyed.items()]
        # positions a request may reach: the model's limit and that of every part (a table's length)
        limits = [model.spec.max_positions] + [p.position_limit() for p in model.all_parts()]
        self.max_positions = min(int(l) for l in limits if l is not None)
        self.cache = CacheManager(self.groups, [self.num_pages] * len(self.groups), self.page_size,
                                  self.max_requests, self.max_positions)
        self.storage = CacheStorage(self.groups, [self.num_pages] * len(self.groups), self.page_size,
                                    self.runtime.dtype, self.device)
        for slot, need in enumerate(needs):
            if need.has_state:
                self.storage.add_state(slot, self.max_requests, need.state_shape, need.state_dtype)
        self._slot_group = {s: g for g, spec in enumerate(self.groups) for s in spec.slots}
        self.has_state = bool(self.storage.state)      # some mixer keeps fixed-size state per request
        self._has_window = any(g.kind == "window" for g in self.groups)

        self.ws = Workspace(self.device)
        self._ring = _PinnedRing()
        self._meta_dev: Optional[torch.Tensor] = None
        # tiles of prompt portions and rows of single tokens are listed for the parts that ask for them
        tile_rows = {int(r) for r in (p.portion_tile_rows() for p in model.all_parts()) if r}
        if len(tile_rows) > 1:
            raise ValueError("parts of the model ask for prompt tiles of different heights: %s" % sorted(tile_rows))
        self._tile_rows = tile_rows.pop() if tile_rows else 0
        self.cu_count = torch.cuda.get_device_properties(self.device).multi_processor_count
        self.steps_run = 0
        # decode steps (one token per request, its logits wanted) replay a captured HIP graph
        self.use_graphs = bool(use_graphs) and all(p.graph_safe for p in model.all_parts())
        self.graph_max_batch = int(graph_max_batch)
        self._graphs: "OrderedDict[tuple, _DecodeGraph]" = OrderedDict()
        self.max_graphs = max(1, int(max_graphs))
        self._graph_ws: Optional[Workspace] = None      # shared by all recorded steps of a natively stepped model
        self.graph_steps = 0         # steps that took the recorded path (the recording one included)
        self.graph_replays = 0       # of these, replays of an existing recording
        self.steps_ahead = 0         # recorded steps that took their tokens from the device (step_ahead)
        self._sample_host = None     # pinned staging of the sampler's per-row parameters, and of its tokens
        self._sampled_host = None
        self._ahead_out = None       # two sets of buffers for tokens sampled without waiting, used in turn
        self._ahead_turn = 0
        self.graphs_evicted = 0
        self.graph_after = max(1, int(graph_after))
        self._graph_seen: "OrderedDict[tuple, int]" = OrderedDict()     # shapes not yet recorded: how often they came
        self.graph_deferred = 0      # decode steps run eagerly because their shape had not come back yet
        # the step function in native code, when the model's parts all have a native description
        from .native import NativeDecoder
        self.native = NativeDecoder.try_build(self) if use_native else None
        self.native_steps = 0

    # ---- construction -----------------------------------------------------------------
    @classmethod
    def from_dir(cls, model_dir: str, dtype=None, device="cuda:0", max_tokens: Optional[int] = None,
                 attention_impl: str = "auto", gemm_impl: str = "auto", max_context: Optional[int] = None,
                 **kw):
        """``dtype`` None: the checkpoint's own (config.json's torch_dtype; float16 runs as bfloat16)."""
        cfg = config_from_dir(model_dir, max_tokens=max_context) if max_context else config_from_dir(model_dir)
        if dtype is None:
            dtype = getattr(torch, getattr(cfg, "default_dtype", "bfloat16"))
        rt = Runtime(dtype=dtype, device=device, attention_impl=attention_impl, gemm_impl=gemm_impl)
        model = build_model(cfg.model_spec(), rt)
        model.load_from_dir(model_dir)
        if max_tokens is None:
            max_tokens = model.spec.max_positions
        eng = cls(model, max_tokens=max_tokens, **kw)
        eng.config = cfg
        return eng

    # ---- requests -------------------------------------------------------------------------
    def has_request(self, req_id) -> bool:
        return self.cache.has_request(req_id)

    def add_request(self, req_id) -> None:
        slot = self.cache.admit(req_id)
        self.storage.zero_state(slot)

    def free(self, req_id) -> None:
        if self.cache.has_request(req_id):
            self.cache.release(req_id)

    def length(self, req_id) -> int:
        return self.cache.length(req_id)

    def fork(self, src_id, dst_id, n_tokens: Optional[int] = None) -> None:
        """A new request ``dst_id`` that holds a copy of the first ``n_tokens`` cached tokens of
        ``src_id`` (all by default) in pages of its own; both go on independently.  What the
        reference's duplicateKVCache does for its slabs (src/models/jiuge/jiuge_kv_cache.cpp:25-47).
        Fixed-size state of ``src_id`` is copied as it is now, so with such state only a full copy
        (``n_tokens`` None or the whole length) is meaningful."""
        slot, pairs = self.cache.fork(src_id, dst_id, n_tokens)
        for g in range(len(self.groups)):
            mine = [(s, d) for gg, s, d in pairs if gg == g]
            self.storage.copy_pages(g, [s for s, _ in mine], [d for _, d in mine])
        if self.storage.state:
            self.storage.copy_state(self.cache.state_slot(src_id), slot)

    def adopt(self, old_id, new_id, n_tokens: int) -> None:
        """``new_id`` takes over the cache of ``old_id`` cut down to its first ``n_tokens`` tokens: a new
        request goes on from the prefix it shares with a finished one (scripts/kvcache_pool.py:18-42)."""
        self.cache.rename(old_id, new_id)
        self.cache.truncate(new_id, n_tokens)

    # ---- the step ----------------------------------------------------------------------------
    def step(self, entries: Sequence[StepEntry]):
        """Run the entries' tokens as one batch.  Returns float32 logits
        [number of wanted places, vocab] on the device, in the order of the entries and
        of each entry's ``want`` (None when nothing is wanted).  The tensor is a
        workspace view: it is valid until the next step."""
        if not entries:
            return None
        if self.use_graphs and len(entries) <= self.graph_max_batch:
            starts = self._append_single_tokens(entries)
            if starts is not None:                   # a pure decode step: the lean way through the same checks
                try:
                    logits = self._graph_step(entries, starts)
                except BaseException:
                    self._forget_recorded_rows()
                    for e, p0 in zip(entries, starts):
                        self.cache.truncate(e.req_id, p0)
                    raise
                if self._has_window:
                    for e in entries:
                        self.cache.trim(e.req_id)
                self.steps_run += 1
                return logits
        vocab = self.model.spec.vocab_size
        seen = set()
        for e in entries:
            if e.req_id in seen:
                raise ValueError("request %r appears twice in one step" % (e.req_id,))
            seen.add(e.req_id)
            if len(e.tokens) == 0:
                raise ValueError("request %r brings no tokens" % (e.req_id,))
            if min(e.tokens) < 0 or max(e.tokens) >= vocab:
                raise ValueError("a token id of request %r is outside the vocabulary (%d): %r"
                                 % (e.req_id, vocab, [t for t in e.tokens if not 0 <= t < vocab][:5]))
            for w in e.want:
                if not (0 <= int(w) < len(e.tokens)):
                    raise ValueError("wanted place %r of request %r is outside its %d tokens" % (w, e.req_id, len(e.tokens)))

        # ---- room in the cache and in the positions: all or nothing -------------------------------
        # Everything that can refuse the step is looked at for ALL entries before anything changes.
        new_ids = [e.req_id for e in entries if not self.cache.has_request(e.req_id)]
        before = {e.req_id: (self.cache.length(e.req_id) if self.cache.has_request(e.req_id) else 0)
                  for e in entries}
        for e in entries:
            if before[e.req_id] + len(e.tokens) > self.max_positions:
                raise PositionOverflow("request %r would reach position %d, the model ends at %d"
                                       % (e.req_id, before[e.req_id] + len(e.tokens), self.max_positions))
        if len(new_ids) > self.cache.slots.n_free:
            raise OutOfPages("%d new requests but %d free state slots" % (len(new_ids), self.cache.slots.n_free))
        need = [0] * len(self.groups)
        for e in entries:
            if self.cache.has_request(e.req_id):
                per = self.cache.pages_needed(e.req_id, len(e.tokens))
            else:
                per = [(len(e.tokens) + self.page_size - 1) // self.page_size] * len(self.groups)
            need = [a + b for a, b in zip(need, per)]
        for g, n in enumerate(need):
            if n > self.cache.free_pages(g):
                raise OutOfPages("step needs %d pages of group %d, %d free" % (n, g, self.cache.free_pages(g)))

        # From here on the cache changes.  Should anything still fail (an allocation, a kernel that
        # refuses its arguments), the cache is put back: lengths, pages and newly admitted requests.
        # What a failed forward wrote lies beyond every request's length and is never read.
        try:
            for rid in new_ids:
                self.add_request(rid)
            starts = [self.cache.append(e.req_id, len(e.tokens)) for e in entries]
            if (self.use_graphs and len(entries) <= self.graph_max_batch
                    and all(len(e.tokens) == 1 and list(e.want) == [0] for e in entries)):
                logits = self._graph_step(entries, starts)
            else:
                with ops.stream_scope():
                    logits = self._eager_step(entries, starts)
        except BaseException:
            self._forget_recorded_rows()
            for e in entries:
                if e.req_id in new_ids:
                    if self.cache.has_request(e.req_id):
                        self.cache.release(e.req_id)
                elif self.cache.length(e.req_id) != before[e.req_id]:
                    self.cache.truncate(e.req_id, before[e.req_id])
            raise
        for e in entries:
            self.cache.trim(e.req_id)
        self.steps_run += 1
        return logits

    def step_ahead(self, entries: Sequence[StepEntry], device_tokens):
        """The next decode step of requests whose last tokens the host has not seen yet: every entry is one admitted
        request's single next token with its logits wanted, its ``tokens`` a placeholder ([0]); the tokens themselves
        are ``device_tokens`` (int32 [len(entries)] on the device, what ``sample_ahead`` returned for the step before,
        in the order of the entries).  Only a recorded step can run so: returns its logits, or None with nothing
        changed when there is no recording for this batch size and context yet, when pages are missing or anything
        else is amiss (the caller then waits for the tokens and calls ``step``)."""
        R = len(entries)
        if (not self.use_graphs or R == 0 or R > self.graph_max_batch or self._has_window
                or device_tokens is None or device_tokens.numel() != R or device_tokens.dtype != torch.int32):
            return None
        reqs = self.cache.requests
        longest = 0
        for e in entries:
            req = reqs.get(e.req_id)
            if req is None:
                return None
            longest = max(longest, req.length)
        g = self._graphs.get((R, _context_bucket(longest + 1)))
        if g is None or g.graph is None:
            return None
        starts = self._append_single_tokens(entries)
        if starts is None:
            return None
        try:
            logits = self._graph_step(entries, starts, device_tokens)
        except BaseException:
            self._forget_recorded_rows()
            for e, p0 in zip(entries, starts):
                self.cache.truncate(e.req_id, p0)
            raise
        self.steps_run += 1
        self.steps_ahead += 1
        return logits

    def _forget_recorded_rows(self):
        """After a step that failed: the pinned images of the recorded steps may hold block-table rows with pages that
        the failed step took and that are given back now.  Such a row is rewritten only when its key (request, page
        count, first live page) changes, and the same key can come back with another page; so every row is
        written anew at its next use."""
        for g in self._graphs.values():
            g.forget_rows()

    def _drop_native(self):
        """The native step function cannot run this model's products (the library has no algorithm for one): from
        now on the parts' forward steps it.  Recordings made around the native call, and the frozen workspace they
        share, go with it."""
        self.native = None
        self._graphs.clear()
        self._graph_ws = None

    def _append_single_tokens(self, entries):
        """The checks and the cache growth of a step in which every entry is an admitted request's single
        next token with its logits wanted, in one pass (a decode step of 64 requests spends as long in
        the general path's per-entry calls as a small model's kernels take).  Returns the tokens'
        positions, or None when the step is not of that kind or anything is amiss: the general path
        then runs, and raises what has to be raised.  Nothing is changed before everything is checked."""
        cache, ps, vocab, limit = self.cache, self.page_size, self.model.spec.vocab_size, self.max_positions
        reqs, pools = cache.requests, cache.pools
        need = [0] * len(pools)
        found = []
        for e in entries:
            toks, want = e.tokens, e.want
            if len(toks) != 1 or len(want) != 1 or want[0] != 0:
                return None
            req = reqs.get(e.req_id)
            if req is None or not (0 <= toks[0] < vocab) or req.length >= limit:
                return None
            found.append(req)
            pages = req.length // ps + 1                  # pages that hold length + 1 tokens
            for g, table in enumerate(req.tables):
                if len(table) < pages:
                    need[g] += pages - len(table)
        if len({id(r) for r in found}) != len(found):
            return None
        for g, n in enumerate(need):
            if n > pools[g].n_free:
                return None
        starts = []
        for req in found:
            pages = req.length // ps + 1
            for g, table in enumerate(req.tables):
                while len(table) < pages:
                    table.append(pools[g].alloc())
            starts.append(req.length)
            req.length += 1
        return starts

    def _eager_step(self, entries, starts):
        """A step that is not a replay: native code lays the batch out and launches it when the model
        allows; otherwise the batch is packed here and the parts' forward runs."""
        from ..parts import linear as _linear
        if self.native is not None and not _linear.TUNE_LIBRARY:
            try:
                out = self.native.step(self, entries, starts)
                self.native_steps += 1
                return out
            except ops.NoLibraryAlgorithm:
                self._drop_native()       # see _forward; nothing of the half-issued step is kept
        return self.model.forward(self._build_context(entries, starts))

    def _forward(self, ctx):
        """The model's forward for a packed step: issued by one native call when the model allows it
        (not while library products are being timed: that is done product by product from Python)."""
        from ..parts import linear as _linear
        if self.native is not None and not _linear.TUNE_LIBRARY:
            try:
                out = self.native.forward(ctx)
                self.native_steps += 1
                return out
            except ops.NoLibraryAlgorithm:
                # the library has no algorithm for a product of this step: the Python path knows a detour.
                # Nothing of the half-issued step is kept (the residual stream is rebuilt, cache writes repeat).
                self._drop_native()
        return self.model.forward(ctx)

    # ---- packing the batch ------------------------------------------------------------------------
    def _build_context(self, entries, starts) -> StepContext:
        ps = self.page_size
        R = len(entries)
        lens = [len(e.tokens) for e in entries]
        T = sum(lens)
        req_start = [0]
        for n in lens:
            req_start.append(req_start[-1] + n)
        want_rows, decode_rows, tiles = [], [], []
        max_ctx = 0
        for r, (e, p0, n) in enumerate(zip(entries, starts, lens)):
            row0 = req_start[r]
            want_rows.extend(row0 + int(w) for w in e.want)
            if n == 1:
                max_ctx = max(max_ctx, p0 + 1)
            if not self._tile_rows:
                continue
            if n == 1:
                decode_rows.append((p0, row0))
            else:
                for o in range(0, n, self._tile_rows):
                    tiles.append((r, row0 + o, min(self._tile_rows, n - o), p0 + o))
        state_slots = [self.cache.state_slot(e.req_id) for e in entries]
        # tiles that see the most keys go first, so the longest blocks do not form the tail; likewise the
        # single tokens (their order is free: each names its row), unless all rows are single tokens and
        # the kernel takes the rows as they lie
        tiles.sort(key=lambda t: -(t[3] + t[2]))
        if len(decode_rows) < T:
            decode_rows.sort(key=lambda pr: -pr[0])
        decode_rows = [row for _, row in decode_rows]

        n_groups = len(self.groups)
        tables = [[self.cache.block_table(e.req_id, g) for e in entries] for g in range(n_groups)]
        group_maxb = [max([1] + [len(t) for t in tables[g]]) for g in range(n_groups)]
        sizes = [("tokens", T), ("positions", T), ("token_req", T), ("state_slots", R),
                 ("want_rows", len(want_rows)), ("decode_rows", len(decode_rows)), ("tiles", 4 * len(tiles))]
        for g in range(n_groups):
            sizes += [("slots%d" % g, T), ("tables%d" % g, R * group_maxb[g])]
        offsets, total = {}, 0
        for name, n in sizes:
            offsets[name] = (total, n)
            total += _align4(n)
        host = self._ring.get(total)
        a = host.numpy()

        def put(name, values):
            o, n = offsets[name]
            a[o:o + n] = values

        for r, (e, p0, n) in enumerate(zip(entries, starts, lens)):     # per request, vectorised over its tokens
            row0 = req_start[r]
            o = offsets["tokens"][0] + row0
            a[o:o + n] = e.tokens
            o = offsets["positions"][0] + row0
            pos = np.arange(p0, p0 + n, dtype=np.int32)
            a[o:o + n] = pos
            o = offsets["token_req"][0] + row0
            a[o:o + n] = r
            for g in range(n_groups):
                table = np.asarray(tables[g][r], dtype=np.int32)
                o = offsets["slots%d" % g][0] + row0
                a[o:o + n] = table[pos // ps] * ps + pos % ps
                o = offsets["tables%d" % g][0] + r * group_maxb[g]
                a[o:o + len(table)] = np.maximum(table, 0)     # pages given back are never read; keep the index valid
                a[o + len(table):o + group_maxb[g]] = 0
        put("state_slots", state_slots)
        put("want_rows", want_rows)
        put("decode_rows", decode_rows)
        if tiles:
            put("tiles", np.asarray(tiles, dtype=np.int32).reshape(-1))
        if self._meta_dev is None or self._meta_dev.numel() < total:
            self._meta_dev = torch.empty(max(total, 4096), dtype=torch.int32, device=self.device)
        dev = self._meta_dev
        dev[:total].copy_(host[:total], non_blocking=True)
        self._ring.mark()

        def view(name):
            o, n = offsets[name]
            return dev[o:o + n]

        ctx = StepContext()
        ctx.T, ctx.R, ctx.page_size, ctx.ws = T, R, ps, self.ws
        ctx.tokens, ctx.positions, ctx.token_req = view("tokens"), view("positions"), view("token_req")
        ctx.state_slots = view("state_slots")
        ctx.want_rows, ctx.n_want = view("want_rows"), len(want_rows)
        ctx.want_rows_identity = (len(want_rows) == T and all(w == i for i, w in enumerate(want_rows)))
        ctx.decode_rows, ctx.n_decode_rows = view("decode_rows"), len(decode_rows)
        ctx.decode_rows_identity = (len(decode_rows) == T and T > 0)
        ctx.prefill_tiles = view("tiles").view(-1, 4)
        ctx.n_prefill_tiles = len(tiles)
        ctx.req_start, ctx.req_pos = req_start, list(starts)
        ctx.req_len = lens
        ctx.req_ids = [e.req_id for e in entries]
        ctx.host_state_slots = state_slots
        ctx.max_position = max(p0 + n - 1 for p0, n in zip(starts, lens))
        ctx.max_context = _context_bucket(max_ctx) if max_ctx else 0
        ctx.cu_count = self.cu_count
        group_views = [(view("slots%d" % g), view("tables%d" % g).view(R, group_maxb[g])) for g in range(n_groups)]
        ctx.group_views = group_views
        for slot in range(self.model.spec.num_cache_slots()):
            state = self.storage.state.get(slot)
            if slot in self._slot_group:
                slots, tables_g = group_views[self._slot_group[slot]]
                ctx._views[slot] = LayerCacheView.of_planes(self.storage.planes(slot), slots, tables_g, state)
            else:
                ctx._views[slot] = LayerCacheView(state=state)
        return ctx

    # ---- decode steps as captured graphs ------------------------------------------------------------
    def _graph_step(self, entries, starts, device_tokens=None):
        """A step of single tokens, one per request, all logits wanted.  The kernels of
        such a step differ from step to step only in the integers they read (tokens,
        positions, slots, block tables), so the launch sequence is captured once per
        (batch size, key split) into a HIP graph with those integers in a fixed device
        buffer, and replayed after one copy into that buffer."""
        R = len(entries)
        bucket = _context_bucket(max(starts) + 1)
        key = (R, bucket)
        g = self._graphs.get(key)
        if g is None and self.graph_after > 1:
            # A shape is recorded when it comes back, not when it first appears: while requests join and leave, most
            # shapes are seen once, and recording costs several steps' time.  Until then its steps run eagerly.
            seen = self._graph_seen.get(key, 0) + 1
            self._graph_seen[key] = seen
            self._graph_seen.move_to_end(key)
            while len(self._graph_seen) > 512:
                self._graph_seen.popitem(last=False)
            if seen < self.graph_after:
                self.graph_deferred += 1
                with ops.stream_scope():
                    return self._eager_step(entries, starts)
            del self._graph_seen[key]
        if g is None:
            while len(self._graphs) >= self.max_graphs:          # the least recently used recording goes
                self._graphs.popitem(last=False)
                self.graphs_evicted += 1
            g = _DecodeGraph(self, R, bucket)
            self._graphs[key] = g
        else:
            self._graphs.move_to_end(key)
        g.fill(self, entries, starts)
        g.meta.copy_(g.host, non_blocking=True)
        g.copied.record()
        if device_tokens is not None:               # (only with a recording at hand: step_ahead has looked)
            g.ctx.tokens.copy_(device_tokens)
        g.ctx.max_position = max(starts)
        g.ctx.req_pos = list(starts)
        g.ctx.req_ids = [e.req_id for e in entries]
        self.graph_steps += 1
        if g.graph is None:
            return g.capture(self)          # the first step of a shape runs eagerly (its result) and is recorded
        g.graph.replay()
        self.graph_replays += 1
        return g.logits

    def _graph_workspace(self) -> Workspace:
        """The workspace of recorded steps.  A natively stepped model needs one buffer whose size is
        known beforehand, so all its recordings share one workspace made for the largest recorded
        batch (only one runs at a time, on one stream): what recordings hold does not grow with their
        number.  Otherwise every recording has a workspace of its own (its buffers are asked for by
        name while it is recorded and must never move afterwards)."""
        if self.native is None:
            return Workspace(self.device)
        if self._graph_ws is None:
            ws = Workspace(self.device)
            ws.buffer("native", (self.native.workspace_bytes_for_decode(self.graph_max_batch),), torch.uint8)
            ws.buffer("logits", (self.graph_max_batch, self.model.spec.vocab_size), torch.float32)
            ws.frozen = True
            self._graph_ws = ws
        return self._graph_ws

    def graph_bytes(self) -> int:
        """Device bytes held for recorded decode steps: workspaces and the steps' integer arrays."""
        seen, total = set(), 0
        for g in self._graphs.values():
            total += g.meta.numel() * 4
            if id(g.ctx.ws) not in seen:
                seen.add(id(g.ctx.ws))
                total += g.ctx.ws.bytes()
        if self._graph_ws is not None and id(self._graph_ws) not in seen:
            total += self._graph_ws.bytes()
        return total

    # ---- library products ----------------------------------------------------------------------------
    def tune_library_products(self, token_counts: Sequence[int]) -> None:
        """Let the library's matrix products for prompt portions of the given token counts use their
        fastest algorithm: one dummy step per count is run in which every library product first times
        the algorithms the library has for its shape on the device and keeps the best.  Between
        timed launches 512 MB of scratch memory are overwritten: in a model every product's weights
        come from memory, not from the cache lines a repeated launch would find.  A step whose
        token count is within an eighth of a timed one takes that one's algorithms; other shapes keep
        the library's first choice and cost nothing.  Optional; results live for this process."""
        from ..parts import linear as _linear
        _linear.TUNE_LIBRARY = True
        _linear.TUNE_FLUSH = torch.empty(512 << 20, dtype=torch.uint8, device=self.device)
        try:
            for n in token_counts:
                rid = ("tune", n)
                self.step([StepEntry(rid, [0] * int(n), [int(n) - 1])])
                self.free(rid)
            torch.cuda.synchronize()
        finally:
            _linear.TUNE_LIBRARY = False
            _linear.TUNE_FLUSH = None

    # ---- sampling --------------------------------------------------------------------------------------
    def sample(self, logits, temperature=None, top_k=None, top_p=None, uniform=None) -> List[int]:
        """Tokens for the rows of ``logits``.  With ``temperature`` None every row is
        argmax; otherwise per-row lists of temperature, top_k, top_p and a uniform draw."""
        R = logits.shape[0]
        out = self.ws.buffer("sampled", (R,), torch.int32)
        if temperature is None:
            ops.argmax(logits, out, self.ws.buffer("argmax_val", (64 * R,), torch.float32),
                       self.ws.buffer("argmax_idx", (64 * R,), torch.int32))
        else:
            # the rows' parameters go through pinned memory into workspace buffers: nothing is allocated per step
            n = max(R, self.graph_max_batch, 1)
            if self._sample_host is None or self._sample_host[0].shape[1] < R:
                self._sample_host = (torch.empty(3, n, dtype=torch.float32, pin_memory=True),
                                     torch.empty(n, dtype=torch.int32, pin_memory=True), torch.cuda.Event())
                self._sample_host[2].record()
            f_host, k_host, copied = self._sample_host
            width = f_host.shape[1]
            copied.synchronize()                        # the copies of the call before have read the pinned buffers
            fa, ka = f_host.numpy(), k_host.numpy()
            fa[0, :R], fa[1, :R], fa[2, :R] = temperature, top_p, uniform
            ka[:R] = top_k
            f = self.ws.buffer("sample_f", (3, width), torch.float32)
            k = self.ws.buffer("sample_k", (width,), torch.int32)
            f.copy_(f_host, non_blocking=True)
            k.copy_(k_host, non_blocking=True)
            copied.record()
            ops.sample(logits, out, f[0, :R], k[:R], f[1, :R], f[2, :R])
        host = self._sampled_host
        if host is None or host.numel() < R:
            host = self._sampled_host = torch.empty(max(R, self.graph_max_batch, 1), dtype=torch.int32, pin_memory=True)
        host[:R].copy_(out, non_blocking=True)
        torch.cuda.current_stream().synchronize()
        return host[:R].tolist()

    def sample_ahead(self, logits, temperature=None, top_k=None, top_p=None, uniform=None):
        """As ``sample``, without waiting for the device: returns (the tokens on the device, int32 [rows], and a
        function that waits for them and returns them as a list).  The device tokens can go straight into
        ``step_ahead``; two sets of buffers are used in turn, so a result stays readable until the call after next."""
        R = logits.shape[0]
        if self._ahead_out is None:
            n = max(self.graph_max_batch, 1)
            self._ahead_out = [dict(tokens=torch.empty(n, dtype=torch.int32, device=self.device),
                                    host=torch.empty(n, dtype=torch.int32, pin_memory=True), done=torch.cuda.Event(),
                                    f=torch.empty(3, n, dtype=torch.float32, device=self.device),
                                    f_host=torch.empty(3, n, dtype=torch.float32, pin_memory=True),
                                    k=torch.empty(n, dtype=torch.int32, device=self.device),
                                    k_host=torch.empty(n, dtype=torch.int32, pin_memory=True)) for _ in range(2)]
            for b in self._ahead_out:
                b["done"].record()
        if R > self._ahead_out[0]["tokens"].numel():
            raise ValueError("sample_ahead takes at most %d rows" % self._ahead_out[0]["tokens"].numel())
        self._ahead_turn ^= 1
        b = self._ahead_out[self._ahead_turn]
        b["done"].synchronize()                     # what this set of buffers held two calls ago has been copied out
        out, host, done = b["tokens"][:R], b["host"], b["done"]
        if temperature is None:
            ops.argmax(logits, out, self.ws.buffer("argmax_val", (64 * R,), torch.float32),
                       self.ws.buffer("argmax_idx", (64 * R,), torch.int32))
        else:
            fa, ka = b["f_host"].numpy(), b["k_host"].numpy()
            fa[0, :R], fa[1, :R], fa[2, :R] = temperature, top_p, uniform
            ka[:R] = top_k
            b["f"].copy_(b["f_host"], non_blocking=True)        # (pinned: the host does not wait for the device)
            b["k"].copy_(b["k_host"], non_blocking=True)
            ops.sample(logits, out, b["f"][0, :R], b["k"][:R], b["f"][1, :R], b["f"][2, :R])
        host[:R].copy_(out, non_blocking=True)
        done.record()

        def wait() -> List[int]:
            done.synchronize()
            return host[:R].tolist()
        return out, wait


class _DecodeGraph:
    """Fixed layout of a decode step's integers for R requests, the step context
    built on views of it, and the captured graph."""

    def __init__(self, engine: "Engine", R: int, ctx_bucket: int):
        self.R = R
        ng = len(engine.groups)
        self.maxb = (engine.model.spec.max_positions + engine.page_size - 1) // engine.page_size
        names = ["tokens", "positions", "token_req", "state_slots", "want_rows"]
        sizes = {n: R for n in names}
        for g in range(ng):
            names += ["slots%d" % g, "tables%d" % g]
            sizes["slots%d" % g] = R
            sizes["tables%d" % g] = R * self.maxb
        self.off, total = {}, 0
        for n in names:
            self.off[n] = total
            total += _align4(sizes[n])
        self.total = total
        self.sizes = sizes
        self.meta = torch.zeros(total, dtype=torch.int32, device=engine.device)
        # the host image of ``meta``: pinned, kept between steps and changed only where the step differs
        self.host = torch.zeros(total, dtype=torch.int32, pin_memory=True)
        self.np = self.host.numpy()
        self.copied = torch.cuda.Event()
        self.copied.record()
        self.np[self.off["token_req"]:self.off["token_req"] + R] = range(R)
        self.np[self.off["want_rows"]:self.off["want_rows"] + R] = range(R)
        self._row_keys = [[None] * R for _ in range(ng)]
        self.graph = None
        self.logits = None

        def view(n):
            return self.meta[self.off[n]:self.off[n] + sizes[n]]

        ctx = StepContext()
        # the recorded launches hold the workspace's addresses, so it must never be regrown
        ctx.T, ctx.R, ctx.page_size, ctx.ws = R, R, engine.page_size, engine._graph_workspace()
        ctx.tokens, ctx.positions, ctx.token_req = view("tokens"), view("positions"), view("token_req")
        ctx.state_slots = view("state_slots")
        ctx.want_rows, ctx.n_want, ctx.want_rows_identity = view("want_rows"), R, True
        ctx.decode_rows, ctx.n_decode_rows, ctx.decode_rows_identity = None, R, True
        ctx.prefill_tiles, ctx.n_prefill_tiles = None, 0
        ctx.req_start = list(range(R + 1))
        ctx.req_len = [1] * R
        ctx.max_context = ctx_bucket
        ctx.cu_count = engine.cu_count
        ctx.group_views = [(view("slots%d" % g), view("tables%d" % g).view(R, self.maxb)) for g in range(ng)]
        for slot in range(engine.model.spec.num_cache_slots()):
            state = engine.storage.state.get(slot)
            if slot in engine._slot_group:
                g = engine._slot_group[slot]
                ctx._views[slot] = LayerCacheView.of_planes(engine.storage.planes(slot), view("slots%d" % g),
                                                            view("tables%d" % g).view(R, self.maxb), state)
            else:
                ctx._views[slot] = LayerCacheView(state=state)
        self.ctx = ctx

    def fill(self, engine, entries, starts):
        """Write this step's integers into the pinned image.  Block-table rows are rewritten
        only when the request in that row, its page count or its first live page changed."""
        self.copied.synchronize()                   # the last copy out of the image is done
        ps, a, o = engine.page_size, self.np, self.off
        cache = engine.cache
        slots = []
        for r, (e, p0) in enumerate(zip(entries, starts)):
            req = cache.requests[e.req_id]
            a[o["tokens"] + r] = e.tokens[0]
            a[o["positions"] + r] = p0
            a[o["state_slots"] + r] = req.state_slot
            slots.append(req.state_slot)
            for g in range(len(engine.groups)):
                table = req.tables[g]
                a[o["slots%d" % g] + r] = table[p0 // ps] * ps + p0 % ps
                key = (req.serial, len(table), req.first_live[g])
                if self._row_keys[g][r] != key:
                    base = o["tables%d" % g] + r * self.maxb
                    a[base:base + len(table)] = table
                    if req.first_live[g]:
                        a[base:base + req.first_live[g]] = 0     # pages given back are never read; keep the index valid
                    a[base + len(table):base + self.maxb] = 0
                    self._row_keys[g][r] = key
        self.ctx.host_state_slots = slots

    def forget_rows(self):
        """Every block-table row of the pinned image is written anew at its next use."""
        for keys in self._row_keys:
            for r in range(len(keys)):
                keys[r] = None

    def capture(self, engine):
        """Run the step once eagerly: that is the step's result, and every buffer then exists.  Then
        record the same launches (recording executes nothing).  The step is therefore computed once,
        also when it is recorded; a part that is ``graph_safe`` need not be idempotent."""
        with ops.stream_scope():
            logits = engine._forward(self.ctx)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        stream = torch.cuda.Stream()
        stream.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(stream):
            with torch.cuda.graph(graph, stream=stream):
                with ops.stream_scope():
                    self.logits = engine._forward(self.ctx)
        torch.cuda.current_stream().wait_stream(stream)
        if self.logits is None or logits is None or self.logits.data_ptr() != logits.data_ptr():
            raise RuntimeError("a recorded step must write its logits where the eager step did")
        self.graph = graph
        return logits
