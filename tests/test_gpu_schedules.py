"""Schedules and shapes that the four replay modes of the tiny models do not reach, each against
the plain implementation: many single-token rows beside prompt portions in one step; the wide
grouped-query shape (16 query heads on a kv head of 128, longrope, an inner size of 8,192); the
benchmark's layer sizes in all four modes and both dtypes; pages of 32 tokens; preemption under
temperature sampling; a step that is refused for its positions; the command line."""
import json
import os
import subprocess
import sys

import pytest
import torch

import helpers as H

pytestmark = pytest.mark.gpu

DTYPES = [("float32", torch.float32, H.FP32_TOL), ("bfloat16", torch.bfloat16, H.BF16_TOL)]
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _folder(tmp_path_factory, tag, cfg, seed, std, norm_std=0.1):
    from infinicore_infer_amd.weights import write_random_model
    folder = os.path.join(str(tmp_path_factory.getbasetemp()), "model_" + tag)
    if not os.path.isdir(folder):
        write_random_model(folder, cfg, seed=seed, std=std, norm_std=norm_std)
    return folder


# ---- (a) more than 16 single-token rows beside two prompt portions ------------------------------------
@pytest.mark.parametrize("dname,dtype,tol", DTYPES)
@pytest.mark.parametrize("name", ["A", "C", "D"])
def test_many_single_tokens_beside_prompt_portions(tmp_path_factory, name, dname, dtype, tol):
    """22 requests decode (one token each, contexts of different lengths, listed out of order) while two
    others bring prompt portions, all in one step: the sorted list of single-token rows, the library
    products and the unfused kernels of a step with more than 16 rows, beside the prompt tiles."""
    from infinicore_infer_amd.engine import Engine
    cfg = H.CONFIGS[name][0]
    folder = H.make_model_dir(tmp_path_factory.getbasetemp(), name)
    n_dec = 22
    max_pos = cfg["max_position_embeddings"]
    lens = [min(max_pos - 8, 2 + (13 * i) % 61 + (40 if i % 5 == 0 else 0)) for i in range(n_dec)]
    requests = {"d%02d" % i: H.random_tokens(cfg["vocab_size"], lens[i] + 3, 900 + i) for i in range(n_dec)}
    requests["p0"] = H.random_tokens(cfg["vocab_size"], min(max_pos, 90), 7)
    requests["p1"] = H.random_tokens(cfg["vocab_size"], 37, 8)
    dec = [k for k in requests if k.startswith("d")]
    steps = [{"step": 0, "end": [], "entries": [{"id": k, "tokens": requests[k][:lens[i]], "want": [lens[i] - 1]}
                                               for i, k in enumerate(dec)]}]
    cuts = {"p0": [0, 30, 61, len(requests["p0"])], "p1": [0, 2, 20, 37]}
    for j in range(3):
        ents = []
        order = [dec, dec[1::2] + dec[0::2], list(reversed(dec))][j]        # the rows in another order each step
        if j == 1:
            ents.append({"id": "p0", "tokens": requests["p0"][cuts["p0"][j]:cuts["p0"][j + 1]],
                         "want": list(range(cuts["p0"][j + 1] - cuts["p0"][j]))})
        for i, k in enumerate(order):
            ents.append({"id": k, "tokens": [requests[k][lens[dec.index(k)] + j]], "want": [0]})
            if i == 10 and j != 1:
                ents.append({"id": "p0", "tokens": requests["p0"][cuts["p0"][j]:cuts["p0"][j + 1]],
                             "want": list(range(cuts["p0"][j + 1] - cuts["p0"][j]))})
        ents.append({"id": "p1", "tokens": requests["p1"][cuts["p1"][j]:cuts["p1"][j + 1]],
                     "want": list(range(cuts["p1"][j + 1] - cuts["p1"][j]))})
        steps.append({"step": j + 1, "end": list(requests) if j == 2 else [], "entries": ents})
    engine = Engine.from_dir(folder, dtype=dtype, max_tokens=(n_dec + 4) * 128, page_size=16, max_requests=n_dec + 2)
    got = H.run_trace(engine, steps)
    ref = H.plain_logits(cfg, H.load_state_dict(folder), requests, dtype == torch.bfloat16)
    assert len(got) == n_dec * 4 + len(requests["p0"]) + len(requests["p1"])
    worst = H.compare(got, ref, tol, "%s %s many single tokens beside portions" % (name, dname))
    print("worst", worst)
    engine.cache.check_invariants()
    assert not engine.cache.requests


# ---- (b) the wide grouped-query shape ----------------------------------------------------------------------
WIDE = dict(model_type="fm9g", vocab_size=1031, hidden_size=4096, num_hidden_layers=2, num_attention_heads=32,
            num_key_value_heads=2, intermediate_size=8192, max_position_embeddings=512, rms_norm_eps=1e-6,
            rope_theta=10000.0, scale_emb=12, dim_model_base=256, scale_depth=1.4, tie_word_embeddings=False,
            eos_token_id=2,
            rope_scaling=dict(type="longrope", original_max_position_embeddings=128,
                              short_factor=[1.0 + 3.0 * i / 63 for i in range(64)],
                              long_factor=[1.0 + 2.0 * ((7 * i) % 64) / 63 for i in range(64)]))


@pytest.mark.parametrize("mode", ["last32", "mixed"])
@pytest.mark.parametrize("dname,dtype,tol", DTYPES)
def test_wide_grouped_query_shape(tmp_path_factory, dname, dtype, tol, mode):
    """Two layers of the 8B-like shape through the engine: 16 query heads on each of 2 kv heads of size
    128, longrope, hidden 4,096, inner size 8,192 (rows of 16 KB in the down projection)."""
    from infinicore_infer_amd.engine import Engine
    folder = _folder(tmp_path_factory, "wide_gqa", WIDE, seed=21, std=0.02)
    requests = {"r%d" % i: H.random_tokens(WIDE["vocab_size"], n, 40 + i) for i, n in enumerate([150, 40, 260, 70])}
    steps, max_tokens = {"last32": H.trace_last_one_by_one, "mixed": H.trace_mixed}[mode](requests)
    engine = Engine.from_dir(folder, dtype=dtype, max_tokens=max_tokens, page_size=64, max_requests=4)
    ref = H.plain_logits(WIDE, H.load_state_dict(folder), requests, dtype == torch.bfloat16)
    worst = H.compare(H.run_trace(engine, steps), ref, tol, "wide shape %s %s" % (dname, mode))
    print("worst", worst)
    engine.cache.check_invariants()


# ---- (c) the benchmark's layer sizes in all four modes -------------------------------------------------------
BENCH2 = dict(model_type="minicpm", vocab_size=1999, hidden_size=2304, num_hidden_layers=2, num_attention_heads=36,
              num_key_value_heads=36, intermediate_size=5760, max_position_embeddings=512, rms_norm_eps=1e-5,
              rope_theta=10000.0, scale_emb=12, dim_model_base=256, scale_depth=1.4, tie_word_embeddings=True,
              eos_token_id=2)


@pytest.mark.parametrize("mode", ["whole", "last32", "chunks", "mixed"])
@pytest.mark.parametrize("dname,dtype,tol", DTYPES)
def test_benchmark_layer_sizes_in_the_four_modes(tmp_path_factory, dname, dtype, tol, mode):
    from infinicore_infer_amd.engine import Engine
    folder = _folder(tmp_path_factory, "bench_layers", BENCH2, seed=31, std=0.02)
    requests = {"r%d" % i: H.random_tokens(BENCH2["vocab_size"], n, 60 + i) for i, n in enumerate([140, 33, 200, 65])}
    maker = {"whole": H.trace_whole, "last32": H.trace_last_one_by_one, "chunks": H.trace_chunks,
             "mixed": H.trace_mixed}[mode]
    steps, max_tokens = maker(requests)
    engine = Engine.from_dir(folder, dtype=dtype, max_tokens=max_tokens, page_size=64, max_requests=4)
    ref = H.plain_logits(BENCH2, H.load_state_dict(folder), requests, dtype == torch.bfloat16)
    worst = H.compare(H.run_trace(engine, steps), ref, tol, "benchmark layers %s %s" % (dname, mode))
    print("worst", worst)
    engine.cache.check_invariants()


# ---- (e) pages of 32 tokens -------------------------------------------------------------------------------------
@pytest.mark.parametrize("dname,dtype,tol", DTYPES)
@pytest.mark.parametrize("name", ["B", "C"])
def test_pages_of_32_tokens(tmp_path_factory, name, dname, dtype, tol):
    from infinicore_infer_amd.engine import Engine
    cfg = H.CONFIGS[name][0]
    folder = H.make_model_dir(tmp_path_factory.getbasetemp(), name)
    requests = {"r%d" % i: H.random_tokens(cfg["vocab_size"], n, 300 + i) for i, n in enumerate([31, 32, 33, 97, 64, 200])}
    ref = H.plain_logits(cfg, H.load_state_dict(folder), requests, dtype == torch.bfloat16)
    for maker in (H.trace_mixed, H.trace_last_one_by_one):
        steps, max_tokens = maker(requests)
        engine = Engine.from_dir(folder, dtype=dtype, max_tokens=max_tokens, page_size=32, max_requests=4)
        assert engine.num_pages == max_tokens // 32
        H.compare(H.run_trace(engine, steps), ref, tol, "%s %s pages of 32 %s" % (name, dname, maker.__name__))
        engine.cache.check_invariants()


# ---- pages are really handed from one request to the next ---------------------------------------------------------
def test_mixed_trace_hands_pages_from_one_request_to_the_next(tmp_path_factory):
    """With a pool smaller than the sum of the requests, a page id must serve two requests in turn:
    the block tables are recorded after every step."""
    from infinicore_infer_amd.engine import Engine, StepEntry
    cfg = H.CONFIGS["B"][0]
    folder = H.make_model_dir(tmp_path_factory.getbasetemp(), "B")
    requests = {"r%d" % i: H.random_tokens(cfg["vocab_size"], n, i) for i, n in enumerate([5, 64, 130, 17, 256, 90])}
    steps, max_tokens = H.trace_mixed(requests)
    assert max_tokens < sum(H.ceil64(len(t)) for t in requests.values())
    engine = Engine.from_dir(folder, dtype=torch.float32, max_tokens=max_tokens, page_size=16, max_requests=4)
    owners = {}
    for rec in steps:
        engine.step([StepEntry(e["id"], e["tokens"], e["want"]) for e in rec["entries"]])
        for rid, req in engine.cache.requests.items():
            for page in req.tables[0]:
                owners.setdefault(page, [])
                if rid not in owners[page]:
                    owners[page].append(rid)
        engine.cache.check_invariants()
        for rid in rec["end"]:
            engine.free(rid)
    shared = {p: o for p, o in owners.items() if len(o) > 1}
    assert shared, "no page was used by two requests"
    assert max(len(o) for o in owners.values()) >= 2 and len(owners) <= engine.num_pages


# ---- a step that is refused for its positions changes nothing -------------------------------------------------------
def test_position_overflow_changes_nothing(tmp_path_factory):
    from infinicore_infer_amd.cache import PositionOverflow
    from infinicore_infer_amd.engine import Engine, StepEntry
    cfg = H.CONFIGS["A"][0]                                   # 128 positions
    folder = H.make_model_dir(tmp_path_factory.getbasetemp(), "A")
    engine = Engine.from_dir(folder, dtype=torch.float32, max_tokens=512, page_size=16, max_requests=3)
    toks = H.random_tokens(256, 128, 1)
    engine.step([StepEntry("x", toks[:40], []), StepEntry("y", toks[:120], [])])
    free, slots = engine.cache.free_pages(0), engine.cache.slots.n_free
    table_x = list(engine.cache.block_table("x", 0))
    # the second entry overflows, the third would be new: nothing of the step may stay
    with pytest.raises(PositionOverflow):
        engine.step([StepEntry("x", toks[40:60], [0]), StepEntry("y", toks[:9], [0]), StepEntry("z", toks[:5], [])])
    assert engine.length("x") == 40 and engine.length("y") == 120 and not engine.has_request("z")
    assert engine.cache.free_pages(0) == free and engine.cache.slots.n_free == slots
    assert engine.cache.block_table("x", 0) == table_x
    with pytest.raises(PositionOverflow):                     # a new request whose prompt alone is too long
        engine.step([StepEntry("w", toks + [1], [])])
    assert not engine.has_request("w") and engine.cache.slots.n_free == slots
    engine.cache.check_invariants()
    # and the requests go on as if nothing had happened
    ref = H.plain_logits(cfg, H.load_state_dict(folder), {"x": toks[:60]}, False)
    got = engine.step([StepEntry("x", toks[40:60], [19])]).float().cpu()
    err = float((got[0].double() - ref["x"][59]).abs().max()) / float(ref["x"].abs().max())
    assert err <= H.FP32_TOL
    # a capped context: the cap bounds the positions, the tables are that long
    capped = Engine.from_dir(folder, dtype=torch.float32, max_tokens=128, page_size=16, max_requests=2, max_context=50)
    assert capped.max_positions == 50
    capped.step([StepEntry("c", toks[:50], [])])
    with pytest.raises(PositionOverflow):
        capped.step([StepEntry("c", [3], [0])])
    assert capped.length("c") == 50


def test_a_failure_inside_the_step_puts_the_cache_back(tmp_path_factory):
    """A kernel that refuses its arguments after the cache has taken the step's pages: lengths, pages
    and newly admitted requests are put back."""
    from infinicore_infer_amd.engine import Engine, StepEntry
    from infinicore_infer_amd.kernels import ops
    folder = H.make_model_dir(tmp_path_factory.getbasetemp(), "A")
    engine = Engine.from_dir(folder, dtype=torch.float32, max_tokens=256, page_size=16, max_requests=3)
    toks = H.random_tokens(256, 60, 2)
    engine.step([StepEntry("x", toks[:20], [])])
    free, slots = engine.cache.free_pages(0), engine.cache.slots.n_free
    real = engine._eager_step

    def broken(entries, starts):
        real(entries, starts)                         # the step's kernels run, then the failure
        raise ops.KernelError("forced failure")
    engine._eager_step = broken
    try:
        with pytest.raises(ops.KernelError):
            engine.step([StepEntry("x", toks[20:50], [0]), StepEntry("n", toks[:33], [0])])
    finally:
        engine._eager_step = real
    assert engine.length("x") == 20 and not engine.has_request("n")
    assert engine.cache.free_pages(0) == free and engine.cache.slots.n_free == slots
    engine.cache.check_invariants()
    ref = H.plain_logits(H.CONFIGS["A"][0], H.load_state_dict(folder), {"x": toks[:50]}, False)
    got = engine.step([StepEntry("x", toks[20:50], [29])]).float().cpu()
    assert float((got[0].double() - ref["x"][49]).abs().max()) / float(ref["x"].abs().max()) <= H.FP32_TOL


# ---- (d) preemption under temperature sampling -------------------------------------------------------------------------
@pytest.mark.parametrize("dname,dtype", [("float32", torch.float32), ("bfloat16", torch.bfloat16)])
def test_preemption_under_temperature_sampling_gives_the_same_tokens(tmp_path_factory, dname, dtype):
    """Requests that lose their pages and are recomputed draw the same numbers and, in float32, see the
    same logits to rounding: the sampled continuation equals the run with plenty of pages."""
    from infinicore_infer_amd.engine import Engine
    from infinicore_infer_amd.engine.scheduler import Scheduler
    from infinicore_infer_amd.engine.tasks import InferTask
    cfg = H.CONFIGS["B"][0]
    folder = H.make_model_dir(tmp_path_factory.getbasetemp(), "B")
    prompts = [H.random_tokens(cfg["vocab_size"], n, 70 + i) for i, n in enumerate([30, 45, 20, 38])]

    def run(pages):
        eng = Engine.from_dir(folder, dtype=dtype, max_tokens=pages * 16, page_size=16, max_requests=4)
        sch = Scheduler(eng, max_batch_tokens=48, chunk_size=32)
        tasks = [InferTask("t%d" % i, p, 256, temperature=0.9, topk=40, topp=0.95, end_tokens=[], seed=5,
                           max_new_tokens=40) for i, p in enumerate(prompts)]
        for t in tasks:
            sch.add(t)
        sch.run()
        eng.cache.check_invariants()
        assert eng.cache.free_pages(0) == pages
        return [t.generated for t in tasks], sch.n_preempted

    plenty, n0 = run(64)
    tight, n1 = run(11)
    assert n0 == 0 and n1 > 0
    assert all(len(g) == 40 for g in plenty)
    if dtype == torch.float32:
        assert tight == plenty
    else:
        # bfloat16: with other requests beside it a row runs through other kernels (more rows, other key splits),
        # and a recomputed prompt runs as portions where it ran token by token before: logits move by rounding,
        # a draw that falls on a boundary of the cumulative distribution may then choose the neighbour, and the
        # continuation differs from there on.  The draws are the same numbers, so the two runs agree until such a
        # boundary is hit: long common beginnings, not equality.
        common = [next((i for i, (x, y) in enumerate(zip(a, b)) if x != y), len(a)) for a, b in zip(tight, plenty)]
        print("tokens in common before the first difference:", common)
        assert sum(common) >= 40 and max(common) >= 20


# ---- decoding one step ahead of the host --------------------------------------------------------------------------------
@pytest.mark.parametrize("native", [True, False])
@pytest.mark.parametrize("temperature", [0.0, 0.8])
def test_decoding_ahead_of_the_host_on_the_engine(tmp_path_factory, temperature, native):
    """``overlap``: recorded decode steps take their input tokens from the sampler's output on the device while the
    host still books the step before.  Six requests of different lengths, one of which ends on an end token (chosen
    from the run without overlap), greedy and with temperature sampling, float32 so that both runs see the same
    logits: the same tokens and finish reasons as without overlap, most decode steps issued ahead, every page back."""
    from infinicore_infer_amd.engine import Engine
    from infinicore_infer_amd.engine.scheduler import Scheduler
    from infinicore_infer_amd.engine.tasks import InferTask
    cfg = H.CONFIGS["A"][0]
    folder = H.make_model_dir(tmp_path_factory.getbasetemp(), "A")
    prompts = [H.random_tokens(cfg["vocab_size"], n, 300 + i) for i, n in enumerate([9, 30, 17, 5, 22, 12])]
    news = [40, 25, 33, 40, 12, 40]

    def run(overlap, end_tokens):
        eng = Engine.from_dir(folder, dtype=torch.float32, max_tokens=6 * 96, page_size=16, max_requests=6, use_native=native)
        sch = Scheduler(eng, max_batch_tokens=64, chunk_size=32, overlap=overlap)
        assert sch.overlap == overlap
        tasks = [InferTask("t%d" % i, p, 256, temperature=temperature, topk=1 if temperature == 0 else 30, topp=0.9,
                           end_tokens=end_tokens, seed=11, max_new_tokens=n) for i, (p, n) in enumerate(zip(prompts, news))]
        for t in tasks[:4]:
            sch.add(t)
        calls = 0
        while sch.has_unfinished() or calls < 12:
            if calls == 11:                       # two more arrive while the others decode ahead
                sch.add(tasks[4]); sch.add(tasks[5])
            sch.step()
            calls += 1
        eng.cache.check_invariants()
        assert eng.cache.free_pages(0) == eng.cache.pools[0].num_pages and sch.n_preempted == 0
        return [(t.generated, t.finish_reason) for t in tasks], sch, eng

    base, _, _ = run(False, [])
    stop = base[0][0][20]                          # the first request will end here
    want, s0, e0 = run(False, [stop])
    got, s1, e1 = run(True, [stop])
    assert got == want
    assert want[0][1] == "stop" and len(want[0][0]) <= 21 and any(r == "length" for _, r in want)
    assert s0.n_ahead == 0 and e0.steps_ahead == 0
    assert s1.n_ahead == e1.steps_ahead and s1.n_ahead >= 20


# ---- the command line ---------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dname", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_command_line_generates_what_the_plain_implementation_does(tmp_path, name, dname):
    from plain_model import plain_generate, round_bf16
    folder = H.make_model_dir(tmp_path, name, seed=6)
    cfg = H.CONFIGS[name][0]
    sd = H.load_state_dict(folder)
    prompts = [H.random_tokens(cfg["vocab_size"], n, 20 + i) for i, n in enumerate([9, 23])]
    env = dict(os.environ, PYTHONPATH=ROOT + os.pathsep + os.environ.get("PYTHONPATH", ""))
    rnd = round_bf16 if dname == "bfloat16" else None
    # one prompt, in the reference's manner: tokens as they come, then the time per step
    cmd = [sys.executable, "-m", "infinicore_infer_amd.minicpm", "--amd", folder, "--dtype", dname,
           "--prompt-ids", ",".join(map(str, prompts[0])), "--max-new-tokens", "7", "--page-size", "16",
           "--chunk-size", "4", "--max-batch-tokens", "6"]
    p = subprocess.run(cmd, capture_output=True, text=True, timeout=300, env=env, cwd=ROOT)
    assert p.returncode == 0, p.stderr[-2000:]
    want = plain_generate(cfg, sd, prompts[0], 7, rnd=rnd)
    stop = [i for i, t in enumerate(want) if t in (cfg["eos_token_id"] if isinstance(cfg["eos_token_id"], list) else [cfg["eos_token_id"]])]
    if stop:
        want = want[:stop[0] + 1]
    line = [l for l in p.stdout.splitlines() if l.startswith("tokens[0]")][0]
    assert [int(t) for t in line.split(":")[1].split()] == want, p.stdout
    assert "Time per step" in p.stdout
    # two prompts together through the scheduler, random weights drawn from a configuration file
    conf = tmp_path / "conf.json"
    conf.write_text(json.dumps(dict(cfg, torch_dtype=dname)))
    cmd = [sys.executable, "-m", "infinicore_infer_amd.causal_lm", "--amd", "--random-weights", "--config", str(conf),
           "--weights-seed", "6", "--weights-std", str(H.CONFIGS[name][1]["std"]),
           "--weights-norm-std", str(H.CONFIGS[name][1]["norm_std"]), "--max-new-tokens", "5",
           "--page-size", "32", "--num-pages", "8", "--chunk-size", "8", "--max-batch-tokens", "12"]
    for pr in prompts:
        cmd += ["--prompt-ids", ",".join(map(str, pr))]
    p = subprocess.run(cmd, capture_output=True, text=True, timeout=300, env=env, cwd=ROOT)
    assert p.returncode == 0, p.stderr[-2000:]
    for i, pr in enumerate(prompts):                  # the same seed and rules as the folder above: the same weights
        want = plain_generate(cfg, sd, pr, 5, rnd=rnd)
        stop = [j for j, t in enumerate(want) if t in ([cfg["eos_token_id"]] if isinstance(cfg["eos_token_id"], int) else cfg["eos_token_id"])]
        if stop:
            want = want[:stop[0] + 1]
        line = [l for l in p.stdout.splitlines() if l.startswith("tokens[%d]" % i)][0]
        assert [int(t) for t in line.split(":")[1].split()] == want, p.stdout
    assert "2 requests" in p.stdout


# ---- the kernels' own rounding to bfloat16 ---------------------------------------------------------------------------------
def test_kernels_round_to_bfloat16_to_nearest_even_and_keep_nan():
    """Values chosen on the rounding boundaries go through the norm kernel (weight 1, a row whose
    factor is exactly 1) and must come out as the nearest bfloat16, ties to even; NaN stays NaN and
    infinity stays infinity.  The embedding kernel must reproduce bfloat16 table entries exactly."""
    from infinicore_infer_amd.kernels import ops
    dev = torch.device("cuda:0")
    import struct

    def f32(bits):
        return struct.unpack("<f", struct.pack("<I", bits))[0]
    # the row's mean square is made exactly 1 + tiny so rsqrt(...) rounds to 1.0f: eps = 0 is not allowed,
    # so the probe values ride in a row dominated by +-1 entries with eps chosen as 2^-60
    probes = [f32(0x3F808000), f32(0x3F818000), f32(0x3F808001), f32(0x3F807FFF), f32(0x3F80FFFF),
              f32(0xBF808000), f32(0xBF818000), 1.0, -1.0, f32(0x00000001), f32(0x3F7FFFFF)]
    want_bits = [0x3F80, 0x3F82, 0x3F81, 0x3F80, 0x3F81, 0xBF80, 0xBF82, 0x3F80, 0xBF80, 0x0000, 0x3F80]
    for d, (val, bits) in [(d, pb) for d in (4096, 1001) for pb in zip(probes, want_bits)]:      # the vector kernel and the general one
        # sum of squares must be exactly d: pair the probe with a partner so that v^2 + p^2 = 2 is not
        # needed; instead scale: use rows of all-ones and apply the probe through the WEIGHT, whose
        # product x * r * w is rounded once at the end
        x = torch.ones(1, d, dtype=torch.float32, device=dev)
        w = torch.ones(d, dtype=torch.float32, device=dev)
        w[7] = val
        out = torch.empty(1, d, dtype=torch.bfloat16, device=dev)
        ops.rmsnorm(x, w, out, 2.0 ** -60)
        got = int(out.view(torch.int16)[0, 7].item()) & 0xFFFF
        assert got == bits, "%r rounded to %#06x, expected %#06x" % (val, got, bits)
        assert int(out.view(torch.int16)[0, 8].item()) & 0xFFFF == 0x3F80
    for d, special in [(d, sp) for d in (4096, 1001) for sp in (float("nan"), float("inf"), float("-inf"))]:
        x = torch.ones(1, d, dtype=torch.float32, device=dev)
        w = torch.ones(d, dtype=torch.float32, device=dev)
        w[3] = special
        out = torch.empty(1, d, dtype=torch.bfloat16, device=dev)
        ops.rmsnorm(x, w, out, 2.0 ** -60)
        v = float(out[0, 3])
        assert (v != v) if special != special else v == special
    # the embedding kernel: bfloat16 table entries times 1.0 arrive exactly, also the largest and smallest
    table = torch.tensor([[f32(0x7F7F0000), f32(0x00800000), -0.0, f32(0x3F810000)] * 4], dtype=torch.float32).to(torch.bfloat16).to(dev)
    xo = torch.empty(1, 16, dtype=torch.float32, device=dev)
    ops.embed(torch.zeros(1, dtype=torch.int32, device=dev), table, xo, 1.0)
    assert torch.equal(xo.view(torch.int32), table.float().view(torch.int32))


# ---- a copy of a request's cache, and going on from a shared prefix ------------------------------------------------------
@pytest.mark.parametrize("dname,dtype,tol", DTYPES)
@pytest.mark.parametrize("name", ["B", "C"])
def test_forked_requests_go_on_independently(tmp_path_factory, name, dname, dtype, tol):
    """Engine.fork copies the first tokens of a request into pages of its own (the reference's
    duplicateKVCache).  The copy, fed other tokens, and the original, fed its own, both match the plain
    implementation; a full copy fed the same token gives the very same logits as the original."""
    from infinicore_infer_amd.engine import Engine, StepEntry
    cfg = H.CONFIGS[name][0]
    folder = H.make_model_dir(tmp_path_factory.getbasetemp(), name)
    eng = Engine.from_dir(folder, dtype=dtype, max_tokens=1024, page_size=16, max_requests=4)
    a = H.random_tokens(cfg["vocab_size"], 90, 1)
    b = a[:53] + H.random_tokens(cfg["vocab_size"], 30, 2)          # shares 53 tokens: the cut lies inside a page
    eng.step([StepEntry("a", a[:70], [])])
    eng.fork("a", "b", 53)
    assert eng.length("b") == 53 and not set(eng.cache.block_table("a", 0)) & set(eng.cache.block_table("b", 0))
    eng.cache.check_invariants()
    got = {}
    la = eng.step([StepEntry("a", a[70:], list(range(20))), StepEntry("b", b[53:], list(range(30)))]).float().cpu()
    for i in range(20):
        got[("a", 70 + i)] = la[i].clone()
    for i in range(30):
        got[("b", 53 + i)] = la[20 + i].clone()
    ref = H.plain_logits(cfg, H.load_state_dict(folder), {"a": a, "b": b}, dtype == torch.bfloat16)
    H.compare(got, ref, tol, "%s %s fork" % (name, dname))
    eng.fork("a", "c")                                              # all of it
    l1 = eng.step([StepEntry("a", [7], [0])]).clone()
    l2 = eng.step([StepEntry("c", [7], [0])]).clone()
    assert torch.equal(l1, l2)
    for r in "abc":
        eng.free(r)
    eng.cache.check_invariants()
    assert eng.cache.free_pages(0) == eng.num_pages


@pytest.mark.parametrize("name", ["A", "C"])
def test_prefix_cache_through_the_entry_point(tmp_path, name):
    """With the prefix cache on, a second prompt that starts like a finished request goes on from the shared
    tokens: fewer tokens are computed, the generated tokens are the plain implementation's (float32)."""
    from plain_model import plain_generate
    from infinicore_infer_amd.minicpm import MiniCPMForCausalLM
    cfg = H.CONFIGS[name][0]
    folder = H.make_model_dir(tmp_path, name, seed=8)
    sd = H.load_state_dict(folder)
    cfg_no_eos = dict(cfg)
    model = MiniCPMForCausalLM(folder, dtype=torch.float32, cache_tokens=512, page_size=16, prefix_cache=True)
    model.eos_token_id = []                                          # the lengths are what the test fixes
    system = H.random_tokens(cfg["vocab_size"], 37, 3)
    p1, p2 = system + [5, 6, 7], system + [9, 8]
    out1 = model.generate_batch([p1], 6)[0]
    assert out1 == plain_generate(cfg_no_eos, sd, p1, 6)
    steps_before = model.engine.steps_run
    out2 = model.generate_batch([p2], 6, chunk_size=4)[0]            # the rest of the prompt is 2 tokens: one portion
    assert out2 == plain_generate(cfg_no_eos, sd, p2, 6)
    sched = model.last_scheduler
    assert sched.n_prefix_hits == 1 and sched.prefix_tokens_reused == 37
    assert model.engine.steps_run - steps_before == 6               # one step for the 2 new prompt tokens, five to decode
    # kept caches are given back with the model
    model._scheduler.release_idle()
    model.engine.cache.check_invariants()
    assert model.engine.cache.free_pages(0) == model.engine.num_pages


# ---- the reference's own generation loop over the Python surface -----------------------------------------------------------
@pytest.mark.parametrize("dname", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_the_reference_loop_over_the_python_surface(tmp_path, name, dname):
    """Generation written as the reference writes it (scripts/jiuge.py:548-586): create_kv_cache, InferTask.bind_kvcache,
    batch_infer_one_round, task.next, drop_kv_cache.  Two tasks step together, as the reference's server batches them
    (scripts/launch_server.py:134-159); a third starts from a duplicated cache (duplicateKVCache, jiuge.h:66-69) and
    must go on exactly as the task it was copied from.  All against the plain implementation."""
    from plain_model import plain_generate, round_bf16
    from infinicore_infer_amd.engine.tasks import InferTask
    from infinicore_infer_amd.minicpm import MiniCPMForCausalLM
    folder = H.make_model_dir(tmp_path, name, seed=8)
    cfg = H.CONFIGS[name][0]
    sd = H.load_state_dict(folder)
    rnd = round_bf16 if dname == "bfloat16" else None
    model = MiniCPMForCausalLM(folder, dtype=getattr(torch, dname), cache_tokens=1024, page_size=16, max_requests=8)
    assert model.max_context_len() == cfg["max_position_embeddings"]
    n_new = 9
    prompts = [H.random_tokens(cfg["vocab_size"], n, 60 + i) for i, n in enumerate([11, 30])]
    tasks = []
    for i, p in enumerate(prompts):
        t = InferTask(i, p, model.max_context_len(), 1.0, 1, 1.0, [])       # topk 1: greedy, the reference's default
        t.bind_kvcache(model.create_kv_cache())
        tasks.append(t)
    outs = [[] for _ in tasks]
    fork_at, forked, forked_out = 4, None, []
    for step in range(n_new):
        out = model.batch_infer_one_round(tasks)
        assert len(out) == len(tasks)
        for i, (t, tok) in enumerate(zip(tasks, out)):
            outs[i].append(int(tok))
            t.next(int(tok))
            assert t.kvcache().tokens == (prompts[i] + outs[i])[:t.pos] and t.finish_reason is None
        if step == fork_at:
            # a second cache with a copy of what task 0's cache holds now; a new task goes on from there
            src = tasks[0]
            copy = model.duplicate_kv_cache(src.kvcache(), src.pos)
            assert copy.tokens == src.kvcache().tokens and copy.data() != src.kvcache().data()
            forked = InferTask("fork", prompts[0] + outs[0], model.max_context_len(), 1.0, 1, 1.0, [])
            forked.bind_kvcache(copy, src.pos)                         # only the token after the copied ones is left to feed
            assert forked.tokens == [outs[0][-1]]
    for step in range(n_new - fork_at - 1):
        tok = int(model.batch_infer_one_round([forked])[0])
        forked_out.append(tok)
        forked.next(tok)
    for i, p in enumerate(prompts):
        assert outs[i] == plain_generate(cfg, sd, p, n_new, rnd=rnd), "task %d" % i
    assert forked_out == outs[0][fork_at + 1:]
    # the finish rules of scripts/infer_task.py:27-36: an end token stops, the position limit ends by length
    t = InferTask("e", prompts[0], model.max_context_len(), 1.0, 1, 1.0, [outs[0][2]])
    t.bind_kvcache(model.create_kv_cache())
    for j in range(outs[0].index(outs[0][2]) + 1):
        assert t.finish_reason is None
        t.next(int(model.batch_infer_one_round([t])[0]))
    assert t.finish_reason == "stop" and t.generated == outs[0][:outs[0].index(outs[0][2]) + 1]
    t2 = InferTask("l", prompts[0], len(prompts[0]) + 1, 1.0, 1, 1.0, [])
    t2.bind_kvcache(model.create_kv_cache())
    t2.next(int(model.batch_infer_one_round([t2])[0]))
    assert t2.finish_reason is None
    t2.next(int(model.batch_infer_one_round([t2])[0]))
    assert t2.finish_reason == "length"
    for task in tasks + [forked, t, t2]:
        model.drop_kv_cache(task.release_kvcache())
        assert task.kvcache() is None
    model.engine.cache.check_invariants()
    assert all(model.engine.cache.free_pages(g) == model.engine.cache.pools[g].num_pages for g in range(len(model.engine.groups)))
    model.destroy_model_instance()
