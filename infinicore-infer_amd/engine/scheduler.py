"""The scheduler above the step function: admits requests, cuts prompts into
portions under a token budget, decodes, finishes and frees.

The reference's only scheduler is the server's worker loop
(scripts/launch_server.py:134-159): it pops up to MAX_BATCH tasks, runs one
inferBatch over them (a new task's whole prompt beside the others' single
tokens), re-queues the unfinished ones and releases the finished ones' caches;
there is no token budget and memory is committed per whole-context slab
(scripts/kvcache_pool.py:18-42).  Here:

  * waiting requests are admitted first come first served while a state slot is
    free and the pages of their first portion are there;
  * every step takes all running requests that decode (one token each) first,
    then prompt portions of at most ``chunk_size`` tokens until
    ``max_batch_tokens`` are spent;
  * with ``prefix_cache`` a finished request's cache is kept, with the tokens it holds, until its
    pages are needed; a new request takes over the kept cache that shares the longest prefix with
    its prompt and starts at min(shared, prompt length - 1), the reference pool's rule
    (scripts/kvcache_pool.py:18-42,58-76).  Kept caches are given up, oldest first, before any
    running request is preempted;
  * when pages run out for a decode token, the most recently admitted running
    request is preempted: its pages and slot are given back and it returns to
    the FRONT of the waiting queue with prompt + generated tokens to be
    recomputed; its random draws depend only on (seed, id, token index), so the
    continuation is the same.  A request that cannot fit even alone finishes
    with finish_reason "length";
  * with ``overlap`` (and an engine that has ``step_ahead`` and ``sample_ahead``) pure decoding runs one step
    ahead of the host: while the device computes a step, the host issues the next one, whose input tokens
    the device takes from its own sampler's output, and only then reads the tokens of the step before.  The
    device then never waits for the host's bookkeeping.  ``step`` returns a step's tokens one call later; what
    cannot be known without the tokens (an end token) is found a step late: that request's extra token is dropped
    and its pages are given back then.  Whenever something else is due (a waiting request, a request that ends
    by length, missing pages, a batch the engine has no recording for) the host waits for the tokens and the
    step after is planned as without overlap.  The tokens are the same with and without.

The scheduler only needs ``engine.cache`` (a CacheManager), ``engine.step``,
``engine.sample``, ``engine.add_request`` and ``engine.free``, so its decisions
are tested on the CPU with a stand-in engine.
"""
from collections import OrderedDict, deque
from dataclasses import dataclass, field
from typing import Deque, Dict, List, Optional, Tuple

from ..cache import OutOfPages
from ..sampling import uniform_draw
from .engine import StepEntry
from .tasks import InferTask


@dataclass
class _Ahead:
    """A step whose sampled tokens the host has not read yet."""
    rows: list                       # the requests whose tokens it samples, in the rows' order
    pos: List[int]                   # each request's cache length after the step
    device_tokens: object            # the tokens on the device
    wait: object                     # waits for them and returns them as a list


@dataclass(eq=False)               # compared by identity: membership tests must not compare token lists
class _Running:
    task: InferTask
    feed: List[int]                  # tokens of this request still to be computed (prompt, or prompt + generated)
    cursor: int = 0                  # how many of ``feed`` are computed
    order: int = 0                   # admission counter (larger = admitted later)

    @property
    def decoding(self) -> bool:
        return self.cursor >= len(self.feed)


class Scheduler:
    def __init__(self, engine, max_batch_tokens: int = 2048, chunk_size: int = 512,
                 max_running: Optional[int] = None, prefix_cache: bool = False, overlap: bool = False):
        if max_batch_tokens < 1 or chunk_size < 1:
            raise ValueError("max_batch_tokens and chunk_size must be positive")
        self.engine = engine
        self.cache = engine.cache
        self.max_batch_tokens = max_batch_tokens
        self.chunk_size = chunk_size
        self.max_running = max_running or self.cache.max_requests
        self.waiting: Deque[_Running] = deque()
        self.running: List[_Running] = []
        self.finished: List[InferTask] = []
        self._admitted = 0
        self.n_preempted = 0
        self.n_steps = 0
        self.last_plan: List[Tuple[object, int, int]] = []     # (id, first position, tokens) of the last step
        # Kept caches of finished requests: only where every key stays available (no window group gives
        # pages back) and no fixed-size state exists (a state cannot be cut back to a prefix).
        self.prefix_cache = (bool(prefix_cache) and all(g.kind == "full" for g in self.cache.groups)
                             and not getattr(engine, "has_state", False))
        # decoding one step ahead of the host: not together with kept caches (a cache would be kept with a token more)
        self.overlap = (bool(overlap) and not self.prefix_cache and hasattr(engine, "step_ahead")
                        and hasattr(engine, "sample_ahead") and getattr(engine, "use_graphs", True))
        # rows a step may have to run ahead: what the engine records (a larger batch has no recording, so
        # ``step_ahead`` would refuse it and ``sample_ahead`` has no buffers for it)
        cap = getattr(engine, "graph_max_batch", None)
        self._ahead_rows = (1 << 30) if cap is None else int(cap)
        self._ahead: Optional[_Ahead] = None
        self.n_ahead = 0                 # steps issued before the tokens of the step before were read
        self.idle: "OrderedDict[object, List[int]]" = OrderedDict()    # kept cache id -> the tokens it holds, oldest first
        self._idle_serial = 0
        self.n_prefix_hits = 0
        self.prefix_tokens_reused = 0

    # ---- queueing -----------------------------------------------------------------
    def add(self, task: InferTask) -> None:
        if not task.prompt:
            raise ValueError("request %r has an empty prompt" % (task.id,))
        self.waiting.append(_Running(task, list(task.prompt)))

    def has_unfinished(self) -> bool:
        return bool(self.waiting or self.running or self._ahead is not None)

    def abort(self, task_id) -> None:
        for r in list(self.running):
            if r.task.id == task_id:
                self._finish(r, "cancel")
        for r in list(self.waiting):
            if r.task.id == task_id:
                self.waiting.remove(r)
                r.task.finish_reason = "cancel"
                self.finished.append(r.task)

    # ---- internals --------------------------------------------------------------------
    def _finish(self, r: _Running, reason: str) -> None:
        r.task.finish_reason = reason
        held = self.cache.length(r.task.id) if self.cache.has_request(r.task.id) else 0
        if self.prefix_cache and reason in ("stop", "length") and held > 0:
            self._idle_serial += 1
            kept = ("kept", self._idle_serial)
            self.engine.adopt(r.task.id, kept, held)          # the cache stays, under a name of its own
            self.idle[kept] = (list(r.task.prompt) + list(r.task.generated))[:held]
        else:
            self.engine.free(r.task.id)
        if r in self.running:
            self.running.remove(r)
        self.finished.append(r.task)

    def _preempt(self, r: _Running) -> None:
        """Give back everything ``r`` holds; it will be recomputed from its tokens."""
        self.engine.free(r.task.id)
        self.running.remove(r)
        r.feed = list(r.task.prompt) + list(r.task.generated)
        r.cursor = 0
        self.waiting.appendleft(r)
        self.n_preempted += 1

    def _evict_idle(self, keep=None) -> bool:
        """Give up the oldest kept cache (not ``keep``); False when there is none."""
        for kept in self.idle:
            if kept != keep:
                del self.idle[kept]
                self.engine.free(kept)
                return True
        return False

    def release_idle(self) -> None:
        """Give up every kept cache."""
        while self._evict_idle():
            pass

    def _best_prefix(self, feed: List[int]):
        """(kept cache id, tokens to reuse) with the longest common prefix, by the reference's rule
        min(shared, len - 1) so that at least one token is left to compute; (None, 0) without a match."""
        best, best_n = None, 0
        for kept, toks in self.idle.items():
            n = 0
            for a, b in zip(feed, toks):
                if a != b:
                    break
                n += 1
            if n > best_n:
                best, best_n = kept, n
        return best, min(best_n, len(feed) - 1)

    def _pages_for_new(self, n_tokens: int) -> List[int]:
        ps = self.cache.page_size
        return [(n_tokens + ps - 1) // ps] * len(self.cache.groups)

    def _fits(self, need: List[int], reserved: List[int]) -> bool:
        return all(n + r <= self.cache.free_pages(g) for g, (n, r) in enumerate(zip(need, reserved)))

    # ---- one step -------------------------------------------------------------------------
    def plan(self) -> List[Tuple[_Running, int]]:
        """Decide which request computes how many tokens in the next step."""
        ngroups = len(self.cache.groups)
        reserved = [0] * ngroups
        budget = self.max_batch_tokens
        plan: List[Tuple[_Running, int]] = []

        # 1. decodes, oldest first; preempt the youngest when pages run out.  The usual case first, in one pass:
        # every decoding request gets its token and the pages for them are there (``running`` is in admission
        # order: requests are appended when admitted and a preempted one is admitted anew).
        decoding = [r for r in self.running if r.decoding]
        if decoding and len(decoding) <= budget:
            ps, reqs = self.cache.page_size, self.cache.requests
            need = [0] * ngroups
            for r in decoding:
                e = reqs[r.task.id]
                pages = e.length // ps + 1
                for g, table in enumerate(e.tables):
                    if len(table) < pages:
                        need[g] += pages - len(table)
            if self._fits(need, reserved):
                reserved = need
                plan = [(r, 1) for r in decoding]
                budget -= len(decoding)
                decoding = []
        for r in sorted(decoding, key=lambda r: r.order):
            if r not in self.running or budget < 1:
                continue
            while True:
                need = self.cache.pages_needed(r.task.id, 1)
                if self._fits(need, reserved):
                    reserved = [a + b for a, b in zip(reserved, need)]
                    plan.append((r, 1))
                    budget -= 1
                    break
                if self._evict_idle():                # kept caches of finished requests go before anyone running
                    continue
                victim = max(self.running, key=lambda x: x.order)
                planned = [p for p in plan if p[0] is victim]
                if planned:                      # a younger request already has its page this step: take it back
                    plan.remove(planned[0])
                    budget += planned[0][1]
                    back = self.cache.pages_needed(victim.task.id, planned[0][1])
                    reserved = [a - b for a, b in zip(reserved, back)]
                if victim is r and len(self.running) == 1:
                    self._finish(r, "length")        # alone and still no room: the cache is too small for it
                    break
                self._preempt(victim)
                if victim is r:
                    break

        # 2. prompt portions of running requests, oldest first
        for r in sorted([r for r in self.running if not r.decoding], key=lambda r: r.order):
            if budget < 1:
                break
            n = min(self.chunk_size, len(r.feed) - r.cursor, budget)
            need = self.cache.pages_needed(r.task.id, n)
            while not self._fits(need, reserved) and self._evict_idle():
                pass
            if not self._fits(need, reserved):
                continue
            reserved = [a + b for a, b in zip(reserved, need)]
            plan.append((r, n))
            budget -= n

        # 3. admissions, first come first served
        while self.waiting and budget >= 1 and len(self.running) < self.max_running:
            r = self.waiting[0]
            if self.cache.max_positions is not None and len(r.feed) > self.cache.max_positions:
                self.waiting.popleft()
                r.task.finish_reason = "length"
                self.finished.append(r.task)
                continue
            kept, shared = self._best_prefix(r.feed) if self.idle else (None, 0)
            if kept is None or shared < 1:
                kept, shared = None, 0
                if self.cache.slots.n_free == 0 and not self._evict_idle():
                    break
            n = min(self.chunk_size, len(r.feed) - shared, budget)
            ps = self.cache.page_size
            have = (shared + ps - 1) // ps                       # pages the kept prefix brings along
            need = [max(0, (shared + n + ps - 1) // ps - have)] * len(self.cache.groups)
            while not self._fits(need, reserved) and self._evict_idle(keep=kept):
                pass
            if not self._fits(need, reserved):
                break
            self.waiting.popleft()
            if kept is not None:
                del self.idle[kept]
                self.engine.adopt(kept, r.task.id, shared)       # go on from the shared prefix
                r.cursor = shared
                self.n_prefix_hits += 1
                self.prefix_tokens_reused += shared
            else:
                self.engine.add_request(r.task.id)
            self._admitted += 1
            r.order = self._admitted
            self.running.append(r)
            reserved = [a + b for a, b in zip(reserved, need)]
            plan.append((r, n))
            budget -= n

        # nothing can move although requests run: make room by preempting the youngest
        if not plan and self.idle and (self.running or self.waiting):
            self.release_idle()                       # kept caches stood in the way
            return self.plan()
        if not plan and self.running:
            victim = max(self.running, key=lambda x: x.order)
            if len(self.running) == 1:
                self._finish(victim, "length")
            else:
                self._preempt(victim)
            return self.plan()
        if not plan and self.waiting and not self.running:
            r = self.waiting.popleft()               # does not fit an empty cache
            r.task.finish_reason = "length"
            self.finished.append(r.task)
            return self.plan()
        return plan

    # ---- one step ahead of the host ---------------------------------------------------------------------
    def _sampling_arguments(self, rows, ahead: int):
        """() for greedy rows, else the per-row lists ``engine.sample`` takes; ``ahead``: tokens of each row that are
        sampled but not yet in ``generated`` (the random draw is a function of the token's index)."""
        tasks = [r.task for r in rows]
        if all(t.temperature == 0 or t.topk == 1 for t in tasks):
            return ()
        return ([t.temperature for t in tasks], [t.topk for t in tasks], [t.topp for t in tasks],
                [uniform_draw(t.seed, t.id, len(t.generated) + ahead) for t in tasks])

    def _ends_by_length(self, t: InferTask, pos: int, n_generated: int) -> bool:
        return (pos >= t.max_tokens or (self.cache.max_positions is not None and pos >= self.cache.max_positions)
                or (t.max_new_tokens is not None and n_generated >= t.max_new_tokens))

    def _take(self, rows, tokens, positions) -> List[Tuple[InferTask, int]]:
        """Book the tokens a step sampled: append, report, finish.  Rows of requests that have ended meanwhile
        (an end token found a step late, a cancellation) are dropped."""
        out: List[Tuple[InferTask, int]] = []
        for r, tok, pos in zip(rows, tokens, positions):
            t = r.task
            if t.finish_reason is not None:
                continue
            t.generated.append(int(tok))
            t.pos = pos
            out.append((t, int(tok)))
            if tok in t.end_tokens:
                self._finish(r, "stop")
            elif self._ends_by_length(t, pos, len(t.generated)):
                self._finish(r, "length")           # the task's own limit, or the model has no position left
        return out

    def _issue_ahead(self, prev: _Ahead) -> Optional[_Ahead]:
        """The step after ``prev`` from the device's own tokens, when it is plain decoding of the same requests
        and nothing else is due; None when the host has to see the tokens first."""
        if self.waiting or len(self.running) != len(prev.rows) or len(prev.rows) > self.max_batch_tokens:
            return None
        for r, mine, pos in zip(prev.rows, self.running, prev.pos):
            t = r.task
            if r is not mine or t.finish_reason is not None or self._ends_by_length(t, pos, len(t.generated) + 1):
                return None
        entries = [StepEntry(r.task.id, [0], [0]) for r in prev.rows]
        first = [self.cache.length(r.task.id) for r in prev.rows]
        logits = self.engine.step_ahead(entries, prev.device_tokens)
        if logits is None:
            return None
        self.last_plan = [(r.task.id, p, 1) for r, p in zip(prev.rows, first)]
        self.n_steps += 1
        self.n_ahead += 1
        dev, wait = self.engine.sample_ahead(logits, *self._sampling_arguments(prev.rows, 1))
        return _Ahead(prev.rows, [p + 1 for p in first], dev, wait)

    def _step_behind(self) -> List[Tuple[InferTask, int]]:
        """A step is on the device whose tokens the host has not read: issue the one after it if that can be done
        without them, then read and book them."""
        prev = self._ahead
        self._ahead = self._issue_ahead(prev)
        return self._take(prev.rows, prev.wait(), prev.pos)

    def step(self) -> List[Tuple[InferTask, int]]:
        """Run one step; returns (task, new token) for every request that got a token (with ``overlap``, while
        decoding runs ahead of the host: the tokens of the step before the one this call issued)."""
        if self._ahead is not None:
            return self._step_behind()
        plan = self.plan()
        if not plan:
            return []
        entries, samplers = [], []
        self.last_plan = []
        for r, n in plan:
            toks = r.feed[r.cursor:r.cursor + n] if not r.decoding else [r.task.generated[-1]]
            last = r.decoding or r.cursor + n == len(r.feed)
            entries.append(StepEntry(r.task.id, toks, [len(toks) - 1] if last else []))
            self.last_plan.append((r.task.id, self.cache.length(r.task.id), len(toks)))
            if last:
                samplers.append(r)
        logits = self.engine.step(entries)
        for r, n in plan:
            if not r.decoding:
                r.cursor += n
        self.n_steps += 1
        if not samplers:
            return []
        positions = [self.cache.length(r.task.id) for r in samplers]
        if (self.overlap and not self.waiting and len(samplers) == len(self.running)
                and len(samplers) <= self._ahead_rows and all(r.decoding for r in self.running)):
            # every running request decodes from here on: do not wait for this step's tokens, the next call
            # issues the step after it first
            dev, wait = self.engine.sample_ahead(logits, *self._sampling_arguments(samplers, 0))
            self._ahead = _Ahead(list(samplers), positions, dev, wait)
            return []
        tokens = self.engine.sample(logits, *self._sampling_arguments(samplers, 0))
        return self._take(samplers, tokens, positions)

    def run(self, on_step=None) -> List[InferTask]:
        """Step until every request has finished.  ``on_step(new, seconds)``, when given, is called
        after every step with its (task, token) pairs and the time the step took on the host clock
        (a step that samples ends with the copy of its tokens to the host, so that is its whole time)."""
        import time
        while self.has_unfinished():
            t0 = time.perf_counter()
            new = self.step()
            if on_step is not None:
                on_step(new, time.perf_counter() - t0)
        done, self.finished = self.finished, []
        return done
