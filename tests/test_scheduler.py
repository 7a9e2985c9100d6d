"""The scheduler's decisions with a stand-in engine (real cache manager, no GPU). (CPU)"""
import hashlib

import pytest

from infinicore_infer_amd.cache import CacheManager, GroupSpec, OutOfPages
from infinicore_infer_amd.engine.scheduler import Scheduler
from infinicore_infer_amd.engine.tasks import InferTask

VOCAB = 50


def _next_token(history):
    h = hashlib.sha256(",".join(map(str, history)).encode()).digest()
    return h[0] % VOCAB


class FakeEngine:
    """Keeps each request's token history and 'predicts' a token that is a pure function of it,
    so a recomputed request must reproduce its continuation.  Checks what the scheduler feeds."""

    def __init__(self, num_pages, page_size=16, max_requests=4, max_positions=None):
        self.cache = CacheManager([GroupSpec("full", 1, 16, None, (0,))], num_pages, page_size, max_requests,
                                  max_positions)
        self.history = {}
        self.steps = []

    def add_request(self, rid):
        self.cache.admit(rid)
        self.history[rid] = []

    def free(self, rid):
        if self.cache.has_request(rid):
            self.cache.release(rid)
            del self.history[rid]

    def adopt(self, old, new, n_tokens):
        self.cache.rename(old, new)
        self.cache.truncate(new, n_tokens)
        self.history[new] = self.history.pop(old)[:n_tokens]

    def step(self, entries):
        assert len({e.req_id for e in entries}) == len(entries)
        rows = []
        for e in entries:
            start = self.cache.append(e.req_id, len(e.tokens))       # raises OutOfPages if the plan was wrong
            assert start == len(self.history[e.req_id])
            self.history[e.req_id].extend(e.tokens)
            for w in e.want:
                rows.append(_next_token(self.history[e.req_id][:start + w + 1]))
        self.steps.append([(e.req_id, len(e.tokens)) for e in entries])
        self.cache.check_invariants()
        return rows

    def sample(self, logits, temperature=None, top_k=None, top_p=None, uniform=None):
        return list(logits)


def _expected(prompt, n, end=()):
    toks, out = list(prompt), []
    for _ in range(n):
        t = _next_token(toks)
        out.append(t)
        toks.append(t)
        if t in end:
            break
    return out


def _task(i, prompt, new, end=()):
    return InferTask(i, prompt, max_tokens=10 ** 6, end_tokens=list(end), max_new_tokens=new)


def test_prompts_are_cut_under_the_token_budget_and_decodes_come_first():
    eng = FakeEngine(num_pages=64)
    s = Scheduler(eng, max_batch_tokens=40, chunk_size=32)
    s.add(_task("a", list(range(70)), 3))
    s.add(_task("b", list(range(10)), 3))
    s.step()
    assert eng.steps[-1] == [("a", 32), ("b", 8)]         # a's portion, then what the budget leaves for b
    s.step()
    assert eng.steps[-1] == [("a", 32), ("b", 2)]
    s.step()
    assert eng.steps[-1] == [("b", 1), ("a", 6)]          # b decodes first, then a's last portion
    while s.has_unfinished():
        s.step()
        assert sum(n for _, n in eng.steps[-1]) <= 40
        ones = [n for _, n in eng.steps[-1]]
        assert ones == sorted(ones)                       # single decode tokens are listed before portions
    done = {t.id: t for t in s.finished}
    assert done["a"].generated == _expected(range(70), 3) and done["b"].generated == _expected(range(10), 3)
    assert done["a"].finish_reason == "length"
    assert eng.cache.free_pages() == 64 and not eng.cache.requests


def test_budget_is_shared_first_come_first_served():
    eng = FakeEngine(num_pages=64)
    s = Scheduler(eng, max_batch_tokens=48, chunk_size=32)
    for i, n in enumerate([20, 20, 20]):
        s.add(_task(i, list(range(n)), 2))
    s.step()
    assert eng.steps[-1] == [(0, 20), (1, 20), (2, 8)]
    s.step()
    assert eng.steps[-1] == [(0, 1), (1, 1), (2, 12)]


def test_end_tokens_and_position_limit():
    eng = FakeEngine(num_pages=16)
    s = Scheduler(eng)
    prompt = [3, 1, 4, 1, 5]
    full = _expected(prompt, 30)
    stop = full[4]
    t1 = InferTask("s", prompt, max_tokens=10 ** 6, end_tokens=[stop], max_new_tokens=30)
    t2 = InferTask("l", prompt, max_tokens=9, end_tokens=[], max_new_tokens=None)
    s.add(t1)
    s.add(t2)
    s.run()
    assert t1.finish_reason == "stop" and t1.generated == full[:full.index(stop) + 1]
    assert t2.finish_reason == "length" and t2.pos == 9 and t2.generated == full[:5]   # scripts/infer_task.py:33


def test_running_out_of_pages_preempts_the_youngest_and_recomputes_the_same_tokens():
    eng = FakeEngine(num_pages=6, page_size=16, max_requests=4)           # 96 token slots
    s = Scheduler(eng, max_batch_tokens=64, chunk_size=32)
    prompts = {"a": list(range(30)), "b": list(range(5, 35)), "c": list(range(9, 39))}
    for k, p in prompts.items():
        s.add(_task(k, p, 40))
    done = s.run()
    assert s.n_preempted > 0
    for t in done:
        assert t.generated == _expected(prompts[t.id], 40), t.id
        assert t.finish_reason == "length"
    assert eng.cache.free_pages() == 6 and eng.cache.slots.n_free == 4
    # the oldest request was never the victim: it was computed exactly once
    fed_a = sum(n for step in eng.steps for rid, n in step if rid == "a")
    assert fed_a == 30 + 39


def test_a_request_too_large_for_the_cache_ends_with_length():
    eng = FakeEngine(num_pages=2, page_size=16)
    s = Scheduler(eng, max_batch_tokens=64, chunk_size=64)
    big = _task("big", list(range(40)), 5)
    ok = _task("ok", list(range(10)), 30)
    s.add(big)
    s.add(ok)
    s.run()
    assert big.finish_reason == "length" and big.generated == []
    assert ok.finish_reason == "length" and ok.generated == _expected(range(10), 30)[:len(ok.generated)]
    assert len(ok.generated) >= 22                      # it ran until the two pages were full
    assert eng.cache.free_pages() == 2


def test_admission_waits_for_slots_and_is_first_come_first_served():
    eng = FakeEngine(num_pages=64, max_requests=2)
    s = Scheduler(eng, max_batch_tokens=256, chunk_size=64)
    for i in range(5):
        s.add(_task(i, list(range(i, i + 6)), 4))
    order = []
    while s.has_unfinished():
        s.step()
        assert len(eng.cache.requests) <= 2
        for rid, _ in eng.steps[-1]:
            if rid not in order:
                order.append(rid)
    assert order == [0, 1, 2, 3, 4]
    assert all(t.generated == _expected(range(t.id, t.id + 6), 4) for t in s.finished)


def test_abort_frees_everything():
    eng = FakeEngine(num_pages=8)
    s = Scheduler(eng)
    s.add(_task("x", list(range(20)), 50))
    s.add(_task("y", list(range(20)), 50))
    s.step()
    s.abort("x")
    s.abort("y")
    assert not s.has_unfinished() and eng.cache.free_pages() == 8
    assert {t.finish_reason for t in s.finished} == {"cancel"}


def test_sampling_draws_do_not_depend_on_preemption():
    from infinicore_infer_amd.sampling import SamplingParams, uniform_draw
    assert uniform_draw(1, "r", 5) == uniform_draw(1, "r", 5) != uniform_draw(1, "r", 6)
    assert 0.0 <= uniform_draw(2, 7, 0) < 1.0
    assert SamplingParams().greedy and SamplingParams(temperature=0.0, topk=50).greedy
    assert not SamplingParams(temperature=0.8, topk=50).greedy
    with pytest.raises(ValueError):
        SamplingParams(topp=1.5)
    for bad in (dict(temperature=-0.5), dict(temperature=float("nan")), dict(topk=-1), dict(topp=-0.1), dict(topk=2.5)):
        with pytest.raises(ValueError):
            SamplingParams(**bad)
        with pytest.raises(ValueError):                  # a request's options are checked when it is made
            InferTask("bad", [1, 2], 10, **bad)


def test_a_task_whose_limit_lies_beyond_the_models_positions_ends_with_length():
    """max_tokens of a task may exceed what the model can hold; decoding stops at the model's last
    position with "length" instead of asking the step for a position that does not exist."""
    eng = FakeEngine(num_pages=16, max_positions=24)
    s = Scheduler(eng, max_batch_tokens=64, chunk_size=8)
    t = InferTask("t", list(range(10)), max_tokens=10 ** 6, end_tokens=[])
    s.add(t)
    s.run()                                              # FakeEngine.step would raise PositionOverflow
    assert t.finish_reason == "length" and t.pos == 24
    assert t.generated == _expected(range(10), 24 - 10 + 1)
    assert eng.cache.free_pages() == 16
    long = InferTask("long", list(range(30)), max_tokens=10 ** 6)     # the prompt alone is too long
    s.add(long)
    s.run()
    assert long.finish_reason == "length" and long.generated == []


def test_command_line_arguments():
    """The command line's surface: the reference's positional form (scripts/jiuge.py:646-677) and the
    options beside it; parsing needs no GPU."""
    from infinicore_infer_amd.causal_lm import _parse
    path, ndev, a = _parse(["--amd", "/m", "1", "--prompt-ids", "1,2", "--prompt-ids", "3", "--max-new-tokens", "4",
                            "--top-k", "5", "--top-p", "0.5", "--chunk-size", "8", "--max-batch-tokens", "16",
                            "--num-pages", "9", "--page-size", "32", "--dtype", "float32"])
    assert (path, ndev) == ("/m", 1)
    assert a.prompt_ids == ["1,2", "3"] and a.max_new_tokens == 4 and a.topk == 5 and a.topp == 0.5
    assert (a.chunk_size, a.max_batch_tokens, a.num_pages, a.page_size, a.dtype) == (8, 16, 9, 32, "float32")
    path, ndev, a = _parse(["--random-weights", "--config", "c.json", "--prompt-len", "12", "--num-prompts", "3",
                            "--topk", "2", "--max-steps", "6"])
    assert path is None and a.random_weights and a.config == "c.json" and a.prompt_len == 12 and a.num_prompts == 3
    assert a.topk == 2 and a.max_new_tokens == 6 and a.dtype is None
    for bad in (["--nvidia", "/m"], [], ["/m", "--random-weights", "--config", "c"], ["--random-weights"],
                ["/m", "--device", "cpu"]):
        with pytest.raises(SystemExit):
            _parse(bad)


def test_a_new_request_goes_on_from_the_prefix_it_shares_with_a_finished_one():
    """The reference's pool keeps finished requests' caches and hands a new task the one with the longest
    common prefix, starting at min(shared, len - 1) (scripts/kvcache_pool.py:18-42,58-76)."""
    eng = FakeEngine(num_pages=32, max_requests=4)
    s = Scheduler(eng, max_batch_tokens=64, chunk_size=64, prefix_cache=True)
    system = list(range(20, 60))                                  # 40 tokens both prompts start with
    a = _task("a", system + [1, 2, 3], 5)
    s.add(a)
    s.run()
    assert a.generated == _expected(system + [1, 2, 3], 5)
    assert len(s.idle) == 1 and eng.cache.free_pages() < 32      # its cache is kept
    kept_tokens = list(s.idle.values())[0]
    assert kept_tokens == (system + [1, 2, 3] + a.generated)[:47]     # the last token's keys were never computed
    fed_before = sum(n for step in eng.steps for _, n in step)
    b = _task("b", system + [7, 8, 9, 10], 6)
    s.add(b)
    s.run()
    assert b.generated == _expected(system + [7, 8, 9, 10], 6)    # FakeEngine checks that positions and history agree
    assert s.n_prefix_hits == 1 and s.prefix_tokens_reused == 40
    fed_b = sum(n for step in eng.steps for _, n in step) - fed_before
    assert fed_b == 4 + 5                                         # only what lies beyond the shared prefix
    # the same prompt again: everything is shared, one token is still computed (its logits are needed)
    c = _task("c", system + [7, 8, 9, 10], 3)
    s.add(c)
    s.run()
    assert c.generated == _expected(system + [7, 8, 9, 10], 3) and s.prefix_tokens_reused == 40 + 43
    # nothing in common: a fresh cache
    d = _task("d", [5, 4, 3], 2)
    s.add(d)
    s.run()
    assert d.generated == _expected([5, 4, 3], 2) and s.n_prefix_hits == 2
    eng.cache.check_invariants()
    s.release_idle()
    assert eng.cache.free_pages() == 32 and eng.cache.slots.n_free == 4 and not eng.cache.requests


def test_kept_caches_are_given_up_before_a_running_request_is_preempted():
    eng = FakeEngine(num_pages=8, page_size=16, max_requests=3)
    s = Scheduler(eng, max_batch_tokens=64, chunk_size=32, prefix_cache=True)
    first = _task("first", list(range(40)), 8)
    s.add(first)
    s.run()
    assert len(s.idle) == 1 and eng.cache.free_pages() == 8 - 3
    prompts = {"x": list(range(100, 130)), "y": list(range(200, 230))}
    for k, p in prompts.items():
        s.add(_task(k, p, 30))                                    # 2 x 60 tokens = 8 pages: the kept cache has to go
    done = s.run()
    assert s.n_preempted == 0
    for t in done:
        assert t.generated == _expected(prompts[t.id], 30)
    eng.cache.check_invariants()
    # kept caches also hold state slots: with all slots kept, a new request still gets in
    s.release_idle()
    for i in range(3):
        s.add(_task("k%d" % i, [i, i + 1], 2))
    s.run()
    assert len(s.idle) == 3 and eng.cache.slots.n_free == 0
    late = _task("late", [9, 9, 9], 2)
    s.add(late)
    s.run()
    assert late.generated == _expected([9, 9, 9], 2)


def test_prefix_cache_stays_off_where_keys_are_given_back():
    from infinicore_infer_amd.cache import CacheManager, GroupSpec
    eng = FakeEngine(num_pages=8)
    eng.cache = CacheManager([GroupSpec("window", 1, 16, 32, (0,))], 8, 16, 4, None)
    assert not Scheduler(eng, prefix_cache=True).prefix_cache
    assert Scheduler(FakeEngine(num_pages=8), prefix_cache=True).prefix_cache


# ---- decoding one step ahead of the host ------------------------------------------------------------------------------
class AheadEngine(FakeEngine):
    """The stand-in engine with the two calls that decoding ahead needs.  Its 'device tokens' are a function that
    yields the tokens, so that a test can see that the scheduler never looked at them before the next step was
    issued.  ``refuse`` makes step_ahead give up now and then, as a real engine does for a batch it has no
    recording of."""

    def __init__(self, *args, refuse=0, **kw):
        super().__init__(*args, **kw)
        self.refuse, self.ahead_calls, self.ahead_steps, self.reads = refuse, 0, 0, []

    def step_ahead(self, entries, device_tokens):
        from infinicore_infer_amd.engine import StepEntry
        self.ahead_calls += 1
        if self.refuse and self.ahead_calls % self.refuse == 0:
            return None
        if sum(self.cache.pages_needed(e.req_id, 1)[0] for e in entries) > self.cache.free_pages(0):
            return None
        assert all(e.tokens == [0] and list(e.want) == [0] for e in entries)
        self.ahead_steps += 1
        self.reads.append("issue")
        return self.step([StepEntry(e.req_id, [t], [0]) for e, t in zip(entries, device_tokens())])

    def sample_ahead(self, logits, temperature=None, top_k=None, top_p=None, uniform=None):
        rows = list(logits)

        def wait():
            self.reads.append("read")
            return rows
        return (lambda: rows), wait


def _run_requests(overlap, num_pages, refuse, arrivals, end=()):
    eng = AheadEngine(num_pages, page_size=16, max_requests=4, refuse=refuse) if overlap else FakeEngine(num_pages, max_requests=4)
    s = Scheduler(eng, max_batch_tokens=40, chunk_size=24, overlap=overlap)
    tasks, calls = [], 0
    pending = sorted(arrivals, key=lambda a: a[0])
    while pending or s.has_unfinished():
        while pending and pending[0][0] <= calls:
            _, name, prompt, new = pending.pop(0)
            tasks.append(_task(name, prompt, new, end))
            s.add(tasks[-1])
        s.step()
        calls += 1
        assert calls < 5000
    eng.cache.check_invariants()
    assert eng.cache.free_pages(0) == num_pages and not eng.history
    return {t.id: (t.generated, t.finish_reason) for t in tasks}, s, eng


@pytest.mark.parametrize("refuse", [0, 3])
@pytest.mark.parametrize("num_pages", [64, 6])
@pytest.mark.parametrize("seed", [5, 7])
def test_decoding_ahead_of_the_host_gives_the_same_tokens(seed, num_pages, refuse):
    """With ``overlap`` the scheduler issues a decode step before it has read the tokens of the step before.  Requests
    that arrive while others decode, end tokens (found a step late: the extra token is dropped), different lengths,
    few pages (preemption) and an engine that refuses now and then: tokens and finish reasons are those of the run
    without overlap, and every page comes back."""
    import random
    rng = random.Random(seed)
    arrivals = [(at, "r%d" % i, [rng.randrange(VOCAB) for _ in range(rng.randint(3, 40))], rng.randint(1, 40))
                for i, at in enumerate([0, 0, 0, 0, 5, 9, 30, 31, 60])]
    end = (7,)
    want, s0, _ = _run_requests(False, num_pages, 0, arrivals, end)
    got, s1, eng = _run_requests(True, num_pages, refuse, arrivals, end)
    assert got == want
    assert any(reason == "stop" for _, reason in want.values()) and any(reason == "length" for _, reason in want.values())
    assert eng.ahead_steps == s1.n_ahead > 0
    if num_pages == 64:
        assert s1.n_ahead >= 15 and s0.n_preempted == s1.n_preempted == 0
    else:
        assert s0.n_preempted > 0 and s1.n_preempted > 0


def test_decoding_ahead_issues_the_next_step_before_it_reads_the_tokens():
    eng = AheadEngine(64, max_requests=4)
    s = Scheduler(eng, max_batch_tokens=64, chunk_size=64, overlap=True)
    for i in range(3):
        s.add(_task("q%d" % i, [1 + i, 2, 3], 12))
    assert len(s.step()) == 0 and eng.reads == []               # the prompts' step: its tokens are not waited for
    for k in range(5):
        out = s.step()
        assert len(out) == 3 and eng.reads[-2:] == ["issue", "read"]      # the step after is on its way first
    assert s.n_ahead == 5 and s.n_steps == 6
    done = s.run()
    assert sorted(len(t.generated) for t in done) == [12, 12, 12]
    assert [t.generated for t in sorted(done, key=lambda t: t.id)] == [_expected([1 + i, 2, 3], 12) for i in range(3)]
    # without the two calls, or with kept caches, the scheduler stays as it was
    assert not Scheduler(FakeEngine(8), overlap=True).overlap
    assert not Scheduler(AheadEngine(8), overlap=True, prefix_cache=True).overlap


def test_more_running_requests_than_the_engine_runs_ahead():
    """An engine records decode steps up to ``graph_max_batch`` rows and its ``sample_ahead`` has buffers for as
    many: with more running requests the scheduler must not ask it to run ahead (the step before has already
    grown every cache, so a refusal there would lose its tokens)."""
    class Capped(AheadEngine):
        graph_max_batch = 2

        def sample_ahead(self, logits, *a, **kw):
            assert len(list(logits)) <= self.graph_max_batch, "asked to run ahead with more rows than it takes"
            return super().sample_ahead(logits, *a, **kw)

    def run(n_requests, overlap):
        eng = Capped(64, max_requests=4)
        s = Scheduler(eng, max_batch_tokens=64, chunk_size=64, overlap=overlap)
        for i in range(n_requests):
            s.add(_task("q%d" % i, [1 + i, 2, 3], (4, 14, 15)[i]))
        done = s.run()
        eng.cache.check_invariants()
        return {t.id: t.generated for t in done}, s

    three, s3 = run(3, True)
    assert three == run(3, False)[0] and len(three) == 3
    assert [len(three["q%d" % i]) for i in range(3)] == [4, 14, 15]
    # three rows never ran ahead; once one request has ended, the two that are left do
    assert 0 < s3.n_ahead <= 10
    two, s2 = run(2, True)
    assert two == run(2, False)[0] and s2.n_ahead >= 8
