"""The engine against the plain implementation, in float32 and bfloat16:
whole requests; most of a request at once and the last 32 tokens one by one;
portions of changing size; mixed batches with so few pages that they are used
again; long decoding; the first tokens of a sequence."""
import pytest
import torch

import helpers as H

pytestmark = pytest.mark.gpu

DTYPES = [("float32", torch.float32, H.FP32_TOL), ("bfloat16", torch.bfloat16, H.BF16_TOL)]
LENGTHS = {"A": [1, 7, 33, 100, 128, 45], "B": [5, 64, 130, 17, 256, 90], "C": [3, 150, 65, 300, 129, 40],
           "D": [2, 200, 31, 384, 64, 129]}


def _requests(name, seed=0):
    cfg = H.CONFIGS[name][0]
    return {"r%d" % i: H.random_tokens(cfg["vocab_size"], n, seed * 100 + i)
            for i, n in enumerate(LENGTHS[name])}


_engines = {}
_plain = {}


def _engine(tmp_path_factory, name, dtype, max_tokens, page_size=16, attention="auto"):
    from infinicore_infer_amd.engine import Engine
    key = (name, dtype, max_tokens, page_size, attention)
    if key not in _engines:
        folder = H.make_model_dir(tmp_path_factory.getbasetemp(), name)
        _engines[key] = (Engine.from_dir(folder, dtype=dtype, max_tokens=max_tokens, page_size=page_size,
                                         max_requests=8, attention_impl=attention), folder)
    return _engines[key]


def _reference(folder, name, requests, bf16):
    key = (name, bf16, tuple(sorted((k, tuple(v)) for k, v in requests.items())))
    if key not in _plain:
        _plain[key] = H.plain_logits(H.CONFIGS[name][0], H.load_state_dict(folder), requests, bf16)
    return _plain[key]


MODES = {
    "whole": H.trace_whole,
    "last32": H.trace_last_one_by_one,
    "chunks": H.trace_chunks,
    "mixed": H.trace_mixed,
}


@pytest.mark.parametrize("mode", list(MODES))
@pytest.mark.parametrize("dname,dtype,tol", DTYPES)
@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
def test_replay_modes(tmp_path_factory, name, dname, dtype, tol, mode):
    requests = _requests(name)
    steps, max_tokens = MODES[mode](requests)
    engine, folder = _engine(tmp_path_factory, name, dtype, max_tokens)
    ref = _reference(folder, name, requests, dtype == torch.bfloat16)
    got = H.run_trace(engine, steps)
    assert len(got) == sum(len(t) for t in requests.values())
    worst = H.compare(got, ref, tol, "%s %s %s" % (name, dname, mode))
    print("worst error %.3g at %s (allowed %.3g)" % (worst[0], worst[1], tol))
    engine.cache.check_invariants()
    assert not engine.cache.requests, "every request was ended"
    for g in range(len(engine.groups)):
        assert engine.cache.free_pages(g) == engine.num_pages


@pytest.mark.parametrize("dname,dtype,tol", DTYPES)
@pytest.mark.parametrize("page_size", [16, 64])
def test_generic_attention_path(tmp_path_factory, dname, dtype, tol, page_size):
    """The general attention kernel alone (tiled kernels off) on the head-size-64 model."""
    requests = _requests("C")
    steps, max_tokens = H.trace_mixed(requests, seed=3)
    engine, folder = _engine(tmp_path_factory, "C", dtype, max_tokens, page_size=page_size, attention="generic")
    ref = _reference(folder, "C", requests, dtype == torch.bfloat16)
    H.compare(H.run_trace(engine, steps), ref, tol, "C %s generic page %d" % (dname, page_size))


@pytest.mark.parametrize("dname,dtype,tol", DTYPES)
def test_long_decoding(tmp_path_factory, dname, dtype, tol):
    """A short prompt, then every further token one by one up to the model's last position."""
    cfg = H.CONFIGS["C"][0]
    toks = H.random_tokens(cfg["vocab_size"], cfg["max_position_embeddings"], 77)
    requests = {"long": toks}
    steps, max_tokens = H.trace_last_one_by_one(requests, tail=len(toks) - 5)
    engine, folder = _engine(tmp_path_factory, "C", dtype, max_tokens)
    ref = _reference(folder, "C", requests, dtype == torch.bfloat16)
    H.compare(H.run_trace(engine, steps), ref, tol, "C %s long decoding" % dname)


@pytest.mark.parametrize("dname,dtype,tol", DTYPES)
@pytest.mark.parametrize("name", ["A", "B"])
def test_first_tokens(tmp_path_factory, name, dname, dtype, tol):
    """Positions 0, 1, 2 fed one by one, and as one portion: the start of a sequence."""
    cfg = H.CONFIGS[name][0]
    toks = H.random_tokens(cfg["vocab_size"], 3, 5)
    engine, folder = _engine(tmp_path_factory, name, dtype, 64)
    ref = _reference(folder, name, {"f": toks}, dtype == torch.bfloat16)
    one = [{"step": i, "entries": [{"id": "f", "tokens": [toks[i]], "want": [0]}], "end": ["f"] if i == 2 else []}
           for i in range(3)]
    H.compare(H.run_trace(engine, one), ref, tol, "first tokens one by one")
    whole = [{"step": 0, "entries": [{"id": "f", "tokens": toks, "want": [0, 1, 2]}], "end": ["f"]}]
    H.compare(H.run_trace(engine, whole), ref, tol, "first tokens as one portion")


@pytest.mark.parametrize("mode", ["last32", "chunks", "mixed"])
@pytest.mark.parametrize("dname,dtype,tol", DTYPES)
@pytest.mark.parametrize("name,gain", [("A", 9.0), ("C", 2.0), ("D", 2.0)])       # scores about two units apart
def test_replay_modes_with_attention_that_picks_its_keys(tmp_path_factory, name, gain, dname, dtype, tol, mode):
    """With weights of a few hundredths every score is near zero and attention is close to a plain mean of the values: a key
    that is skipped, read from a neighbour's page or seen one position off would move the logits less than the tolerance.
    Here the q and k projections are scaled up until the scores are about two units apart (much more and attention
    turns into an argmax, which two correct bfloat16 computations resolve differently), so that every query picks a few
    keys and what it picks depends on the rotation and on the exact position (and the values are scaled up so that what
    attention adds weighs in the logits); then the replay modes again (single tokens
    after a prompt, portions down to two tokens, mixed batches on pages that are used again)."""
    import os
    from safetensors.torch import save_file
    from infinicore_infer_amd.engine import Engine
    base = H.make_model_dir(tmp_path_factory.getbasetemp(), name)
    folder = os.path.join(str(tmp_path_factory.getbasetemp()), "model_%s_peaked" % name)
    if not os.path.isdir(folder):
        os.makedirs(folder)
        # (and the value projection by 4: in these tiny models the embedding dominates the residual stream, and what
        # attention adds would otherwise move the logits by a few per cent at most)
        sd = {k: ((v.float() * (gain if ("q_proj" in k or "k_proj" in k) else 4.0 if "v_proj" in k else 1.0)).to(v.dtype)).contiguous()
              for k, v in H.load_state_dict(base).items()}
        save_file(sd, os.path.join(folder, "model.safetensors"), metadata={"format": "pt"})
        with open(os.path.join(base, "config.json")) as f, open(os.path.join(folder, "config.json"), "w") as g:
            g.write(f.read())
    cfg = H.CONFIGS[name][0]
    sd = H.load_state_dict(folder)
    requests = _requests(name, seed=3)
    steps, max_tokens = MODES[mode](requests)
    engine = Engine.from_dir(folder, dtype=dtype, max_tokens=max_tokens, page_size=16, max_requests=8)
    ref = H.plain_logits(cfg, sd, requests, dtype == torch.bfloat16)
    # the attention really is peaked: the plain model with the values of every other key swapped gives other logits
    # (checked once, on the longest request, in float32)
    if mode == "last32" and dtype == torch.float32:
        flat = H.plain_logits(cfg, H.load_state_dict(base), {"r3": requests["r3"]}, False)["r3"]
        assert float((flat - ref["r3"]).abs().max()) / float(ref["r3"].abs().max()) > 0.05
    worst = H.compare(H.run_trace(engine, steps), ref, tol, "%s %s %s, peaked attention" % (name, dname, mode), steps=steps)
    print("worst", worst)
    engine.cache.check_invariants()


@pytest.mark.parametrize("dname,dtype,tol", DTYPES)
@pytest.mark.parametrize("name", ["A", "C"])
def test_decoding_twenty_requests_at_once(tmp_path_factory, name, dname, dtype, tol):
    """More rows than the few-row kernels take (16): the prompts of twenty requests in one step, then
    every request's next token in one step, eight times over (library products, the unfused
    norm, rotary and activation kernels, a recorded graph of that batch size)."""
    from infinicore_infer_amd.engine import Engine
    cfg = H.CONFIGS[name][0]
    folder = H.make_model_dir(tmp_path_factory.getbasetemp(), name)
    n_req, n_dec = 20, 8
    lens = [3 + (7 * i) % 41 for i in range(n_req)]
    requests = {"m%d" % i: H.random_tokens(cfg["vocab_size"], lens[i] + n_dec, 500 + i) for i in range(n_req)}
    steps = [{"step": 0, "end": [],
              "entries": [{"id": k, "tokens": t[:lens[i]], "want": [lens[i] - 1]} for i, (k, t) in enumerate(requests.items())]}]
    for j in range(n_dec):
        steps.append({"step": j + 1, "end": list(requests) if j == n_dec - 1 else [],
                      "entries": [{"id": k, "tokens": [t[lens[i] + j]], "want": [0]} for i, (k, t) in enumerate(requests.items())]})
    engine = Engine.from_dir(folder, dtype=dtype, max_tokens=n_req * 64, page_size=16, max_requests=n_req)
    got = H.run_trace(engine, steps)
    ref = H.plain_logits(cfg, H.load_state_dict(folder), requests, dtype == torch.bfloat16)
    assert len(got) == n_req * (1 + n_dec)
    H.compare(got, ref, tol, "%s %s twenty requests" % (name, dname))
    # the shape runs eagerly when it first appears, is recorded when it comes back, and is replayed from then on
    assert engine.graph_deferred == 1 and engine.graph_steps == n_dec - 1 and engine.graph_replays == n_dec - 2
    engine.cache.check_invariants()


@pytest.mark.parametrize("native", [True, False])
def test_fourteen_rows_of_16_kb_go_through_the_sliced_product(tmp_path_factory, native):
    """13..16 rows whose down projection reads rows of 16 KB (intermediate 8,192): that product runs as slices over K with
    the kernel that sums them, adds the residual and norms, while the O projection (rows of 2 KB) keeps the few-row
    kernel with the norm split over two products.  Fourteen requests decode together, bfloat16, against the plain model."""
    from infinicore_infer_amd.engine import Engine
    from infinicore_infer_amd.kernels import ops
    from infinicore_infer_amd.weights import write_random_model
    import os
    cfg = dict(model_type="minicpm", vocab_size=1003, hidden_size=1024, num_hidden_layers=2, num_attention_heads=8,
               num_key_value_heads=2, intermediate_size=8192, max_position_embeddings=256, rms_norm_eps=1e-5,
               rope_theta=10000.0, scale_emb=4, dim_model_base=256, scale_depth=1.4, tie_word_embeddings=False, eos_token_id=2)
    assert ops.gemm_splitk_pays(14, 1024, 8192) and not ops.gemm_splitk_pays(14, 1024, 1024) and not ops.gemm_splitk_pays(12, 1024, 8192)
    folder = os.path.join(str(tmp_path_factory.getbasetemp()), "model_long_rows")
    if not os.path.exists(os.path.join(folder, "model.safetensors")):
        write_random_model(folder, cfg, seed=21, std=0.02)
    n_req, n_dec = 14, 4
    lens = [2 + (5 * i) % 23 for i in range(n_req)]
    requests = {"s%d" % i: H.random_tokens(cfg["vocab_size"], lens[i] + n_dec, 900 + i) for i in range(n_req)}
    steps = [{"step": 0, "end": [],
              "entries": [{"id": k, "tokens": t[:lens[i]], "want": [lens[i] - 1]} for i, (k, t) in enumerate(requests.items())]}]
    for j in range(n_dec):
        steps.append({"step": j + 1, "end": list(requests) if j == n_dec - 1 else [],
                      "entries": [{"id": k, "tokens": [t[lens[i] + j]], "want": [0]} for i, (k, t) in enumerate(requests.items())]})
    engine = Engine.from_dir(folder, dtype=torch.bfloat16, max_tokens=n_req * 64, page_size=16, max_requests=n_req, use_native=native)
    got = H.run_trace(engine, steps)
    ref = H.plain_logits(cfg, H.load_state_dict(folder), requests, True)
    assert len(got) == n_req * (1 + n_dec)
    H.compare(got, ref, H.BF16_TOL, "fourteen requests, long rows, native %s" % native)
    engine.cache.check_invariants()


@pytest.mark.parametrize("n_req", [20, 40])
def test_seventeen_to_sixty_four_rows_at_a_width_where_the_slices_pay(tmp_path_factory, n_req):
    """20 and 40 requests decode together on two layers of the benchmark's sizes, where the O and the down projection
    both run as slices over K (hidden 2,304, inner size 5,760): sliced O with the whole norm applied, the gate/up product fed fully normed rows
    (with the SwiGLU epilogue at 20 rows, the library's product and the activation kernel at 40), sliced down, and the
    head fed normed rows.  The logits equal the plain model's, and the step issued by native code and the one issued
    by the parts' Python forward launch the same kernels: their logits are equal to the bit."""
    from infinicore_infer_amd.engine import Engine, StepEntry
    from infinicore_infer_amd.kernels import ops
    from infinicore_infer_amd.weights import write_random_model
    import os
    cfg = dict(model_type="minicpm", vocab_size=1999, hidden_size=2304, num_hidden_layers=2, num_attention_heads=36,
               num_key_value_heads=36, intermediate_size=5760, max_position_embeddings=256, rms_norm_eps=1e-5,
               rope_theta=10000.0, scale_emb=12, dim_model_base=256, scale_depth=1.4, tie_word_embeddings=True, eos_token_id=2)
    assert ops.gemm_splitk_pays(n_req, 2304, 5760) and ops.gemm_splitk_pays(n_req, 2304, 2304)
    folder = os.path.join(str(tmp_path_factory.getbasetemp()), "model_bench_rows")
    if not os.path.exists(os.path.join(folder, "model.safetensors")):
        write_random_model(folder, cfg, seed=23, std=0.02, norm_std=0.1)
    n_dec = 3
    lens = [2 + (5 * i) % 23 for i in range(n_req)]
    requests = {"s%d" % i: H.random_tokens(cfg["vocab_size"], lens[i] + n_dec, 900 + i) for i in range(n_req)}
    steps = [{"step": 0, "end": [],
              "entries": [{"id": k, "tokens": t[:lens[i]], "want": [lens[i] - 1]} for i, (k, t) in enumerate(requests.items())]}]
    for j in range(n_dec):
        steps.append({"step": j + 1, "end": list(requests) if j == n_dec - 1 else [],
                      "entries": [{"id": k, "tokens": [t[lens[i] + j]], "want": [0]} for i, (k, t) in enumerate(requests.items())]})
    ref = H.plain_logits(cfg, H.load_state_dict(folder), requests, True)
    got = {}
    for native in (True, False):
        engine = Engine.from_dir(folder, dtype=torch.bfloat16, max_tokens=n_req * 64, page_size=16, max_requests=n_req,
                                 use_native=native, use_graphs=False)
        assert (engine.native is not None) == native
        got[native] = H.run_trace(engine, steps)
        assert len(got[native]) == n_req * (1 + n_dec)
        H.compare(got[native], ref, H.BF16_TOL, "%d requests at width 2,304, native %s" % (n_req, native), steps=steps)
        engine.cache.check_invariants()
    assert set(got[True]) == set(got[False])
    for key in got[True]:
        assert torch.equal(got[True][key], got[False][key]), "native and Python-issued steps differ at %r" % (key,)


def test_out_of_pages_changes_nothing(tmp_path_factory):
    from infinicore_infer_amd.cache import OutOfPages
    from infinicore_infer_amd.engine import StepEntry
    engine, _ = _engine(tmp_path_factory, "A", torch.float32, 64)
    toks = H.random_tokens(256, 60, 1)
    engine.step([StepEntry("x", toks, [])])
    with pytest.raises(OutOfPages):
        engine.step([StepEntry("x", [1], [0]), StepEntry("y", toks[:20], [])])
    assert engine.length("x") == 60 and not engine.has_request("y")
    engine.cache.check_invariants()
    engine.free("x")


def test_bad_tokens_are_refused(tmp_path_factory):
    from infinicore_infer_amd.engine import StepEntry
    engine, _ = _engine(tmp_path_factory, "A", torch.float32, 64)
    with pytest.raises(ValueError):
        engine.step([StepEntry("z", [256], [0])])
    with pytest.raises(ValueError):
        engine.step([StepEntry("z", [1, 2], [2])])
    assert not engine.has_request("z")


@pytest.mark.parametrize("dname,dtype,tol", DTYPES)
def test_recorded_decode_steps_equal_eager_ones(tmp_path_factory, dname, dtype, tol):
    """Decode steps replay a recorded graph.  Every replay is checked against the same step run
    eagerly by a second engine, with eager work (prompt portions, synchronising copies) between
    the replays, for two batch sizes and across a change of the key-split bucket."""
    from infinicore_infer_amd.engine import Engine, StepEntry
    folder = H.make_model_dir(tmp_path_factory.getbasetemp(), "C")
    a = Engine.from_dir(folder, dtype=dtype, max_tokens=1024, page_size=16, max_requests=4, use_graphs=True, graph_after=1)
    b = Engine.from_dir(folder, dtype=dtype, max_tokens=1024, page_size=16, max_requests=4, use_graphs=False)
    prompts = {"p": H.random_tokens(331, 250, 1), "q": H.random_tokens(331, 40, 2), "r": H.random_tokens(331, 90, 3)}
    for eng in (a, b):
        eng.step([StepEntry("p", prompts["p"], []), StepEntry("q", prompts["q"], [])])
    toks = H.random_tokens(331, 40, 9)
    for i in range(12):                      # two requests; "p" crosses 256 keys: a new bucket, a new graph
        la = a.step([StepEntry("p", [toks[i]], [0]), StepEntry("q", [toks[i + 1]], [0])]).clone()
        lb = b.step([StepEntry("p", [toks[i]], [0]), StepEntry("q", [toks[i + 1]], [0])]).clone()
        assert torch.equal(la, lb), "replay %d differs from the eager step" % i
        if i == 5:                           # eager work in between: a third request's prompt
            for eng in (a, b):
                eng.step([StepEntry("r", prompts["r"], [])])
    for i in range(6):                       # three requests
        ents = [StepEntry(k, [toks[20 + i + j]], [0]) for j, k in enumerate("pqr")]
        assert torch.equal(a.step(ents).clone(), b.step(ents).clone())
    assert a.graph_steps == 18 and b.graph_steps == 0 and len(a._graphs) >= 3 and a.graph_replays == 18 - len(a._graphs)


@pytest.mark.parametrize("shape", ["2b", "1b", "8b"])
def test_recorded_steps_with_library_products_equal_eager_ones(tmp_path_factory, shape):
    """From 17 rows on a decode step's matrix products are the library's, and they are recorded into
    the graph with everything else.  Two layers of each benchmark shape, bfloat16, 20 and 64
    requests: every replay against the same step run eagerly by a second engine, with eager work
    (a prompt, synchronising copies) between the replays."""
    from infinicore_infer_amd.engine import Engine, StepEntry
    from infinicore_infer_amd.weights import write_random_model
    import os
    sizes = {"2b": dict(hidden_size=2304, num_attention_heads=36, num_key_value_heads=36, intermediate_size=5760),
             "1b": dict(hidden_size=1536, num_attention_heads=24, num_key_value_heads=8, intermediate_size=3840),
             "8b": dict(hidden_size=4096, num_attention_heads=32, num_key_value_heads=2, intermediate_size=16384)}[shape]
    cfg = dict(model_type="minicpm", vocab_size=20011, num_hidden_layers=2, max_position_embeddings=512,
               rms_norm_eps=1e-5, rope_theta=10000.0, scale_emb=12, dim_model_base=256, scale_depth=1.4,
               tie_word_embeddings=True, eos_token_id=2, **sizes)
    folder = os.path.join(str(tmp_path_factory.getbasetemp()), "model_%s_shaped_graph" % shape)
    write_random_model(folder, cfg, seed=11, std=0.02)
    kw = dict(dtype=torch.bfloat16, max_tokens=64 * 128, page_size=64, max_requests=65)
    a = Engine.from_dir(folder, use_graphs=True, graph_after=1, **kw)
    b = Engine.from_dir(folder, use_graphs=False, **kw)
    if shape == "2b":                        # with the algorithms that timing chooses for these row counts (kept per process)
        a.tune_library_products([64, 20])
    ids = ["r%d" % i for i in range(64)]
    for eng in (a, b):
        for i, rid in enumerate(ids):
            eng.step([StepEntry(rid, H.random_tokens(20011, 5 + i % 40, i), [])])
    toks = H.random_tokens(20011, 200, 77)
    for n_req in (64, 20):
        for i in range(5):
            ents = [StepEntry(rid, [toks[(7 * i + j) % 200]], [0]) for j, rid in enumerate(ids[:n_req])]
            la, lb = a.step(ents).clone(), b.step(ents).clone()
            assert torch.equal(la, lb), "%d requests: replay %d differs from the eager step" % (n_req, i)
            if i == 2:                       # eager work in between
                for eng in (a, b):
                    eng.step([StepEntry("extra%d" % n_req, H.random_tokens(20011, 33, 5), [32])])
                    eng.free("extra%d" % n_req)
    assert a.graph_steps == 10 and a.graph_replays == 8 and b.graph_steps == 0


def _random_configuration(seed):
    """A tiny configuration drawn from the seed: head sizes in steps of 16, any number of kv heads and of
    query heads on each, widths and inner sizes that are multiples of 8, of 4, of 2, or odd."""
    import random
    rng = random.Random(seed)
    dh = rng.choice([16, 32, 48, 64, 80, 96, 112, 128])
    nkvh = rng.choice([1, 2, 3, 5])
    nh = nkvh * rng.choice([1, 1, 2, 3, 4, 7])
    d = rng.choice([nh * dh, 8 * rng.randint(5, 40), 4 * rng.randint(11, 60), 2 * rng.randint(21, 99), rng.randint(40, 300)])
    di = rng.choice([8 * rng.randint(6, 50), 4 * rng.randint(13, 90), rng.randint(50, 400)])
    max_pos = rng.choice([64, 128, 200, 320])
    cfg = dict(model_type=rng.choice(["minicpm", "fm9g"]), vocab_size=rng.randint(50, 700), hidden_size=d,
               num_hidden_layers=rng.randint(1, 3), num_attention_heads=nh, num_key_value_heads=nkvh, head_dim=dh,
               intermediate_size=di, max_position_embeddings=max_pos, rms_norm_eps=rng.choice([1e-5, 1e-6, 1e-3]),
               rope_theta=rng.choice([1e4, 1e6, 5e4]), scale_emb=rng.choice([1.0, 12, 4.0]),
               dim_model_base=rng.choice([d, max(1, d // 4)]), scale_depth=rng.choice([1.0, 1.4, 2.0]),
               tie_word_embeddings=rng.random() < 0.5, eos_token_id=2)
    if rng.random() < 0.3:
        cfg["rope_scaling"] = dict(type="longrope", original_max_position_embeddings=max_pos // 2,
                                   short_factor=[1.0 + 0.05 * i for i in range(dh // 2)],
                                   long_factor=[1.0 + 0.09 * i for i in range(dh // 2)])
    lens = [min(max_pos, n) for n in (rng.randint(1, max_pos), rng.randint(1, 40), 65, 17)]
    return cfg, lens, rng.choice([16, 64])


@pytest.mark.parametrize("seed", [3, 11, 29, 176, 251, 301, 412, 733])
def test_random_configurations(tmp_path_factory, seed):
    """Configurations nobody chose: each request's last tokens one by one and a mixed trace, in both
    dtypes, against the plain implementation."""
    from infinicore_infer_amd.engine import Engine
    from infinicore_infer_amd.weights import write_random_model
    import os
    cfg, lens, page = _random_configuration(seed)
    folder = os.path.join(str(tmp_path_factory.getbasetemp()), "model_random_%d" % seed)
    write_random_model(folder, cfg, seed=seed, std=min(0.05, cfg["hidden_size"] ** -0.5), norm_std=0.1)
    sd = H.load_state_dict(folder)
    requests = {"r%d" % i: H.random_tokens(cfg["vocab_size"], n, seed * 13 + i) for i, n in enumerate(lens)}
    for dname, dtype, tol in DTYPES:
        ref = H.plain_logits(cfg, sd, requests, dtype == torch.bfloat16)
        for maker in (H.trace_last_one_by_one, H.trace_mixed):
            steps, max_tokens = maker(requests)
            engine = Engine.from_dir(folder, dtype=dtype, max_tokens=max(max_tokens, 64), page_size=page, max_requests=8)
            H.compare(H.run_trace(engine, steps), ref, tol, "seed %d %s %s %r" % (seed, dname, maker.__name__, cfg))
            engine.cache.check_invariants()


def test_trace_run_program(tmp_path):
    """bin/trace_run as a program: files, 'done' lines, exit status, and the logits themselves."""
    import json, os, subprocess, sys
    import numpy as np
    folder = H.make_model_dir(tmp_path, "A", seed=2)
    cfg = H.CONFIGS["A"][0]
    requests = {"a": H.random_tokens(256, 50, 1), "b": H.random_tokens(256, 21, 2)}
    steps, max_tokens = H.trace_mixed(requests, sizes=(9, 2, 5))
    steps[1]["entries"][0]["want"] = []                       # a step entry that wants nothing
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    for dname, tol in (("float32", H.FP32_TOL), ("bfloat16", H.BF16_TOL)):
        out = tmp_path / ("out_" + dname)
        p = subprocess.run([os.path.join(root, "bin", "trace_run"), "--model", folder, "--dtype", dname,
                            "--out", str(out), "--max-tokens", str(max_tokens)],
                           input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True,
                           timeout=300)
        assert p.returncode == 0, p.stderr[-2000:]
        assert p.stdout.split("\n")[:-1] == ["done %d" % s["step"] for s in steps]
        ref = H.plain_logits(cfg, H.load_state_dict(folder), requests, dname == "bfloat16")
        cursor, got = {}, {}
        for s in steps:
            n_want = sum(len(e["want"]) for e in s["entries"])
            path = out / ("%d.f32" % s["step"])
            assert path.exists() == (n_want > 0)
            rows = np.fromfile(path, dtype="<f4").reshape(n_want, 256) if n_want else None
            i = 0
            for e in s["entries"]:
                for w in e["want"]:
                    got[(e["id"], cursor.get(e["id"], 0) + w)] = torch.from_numpy(rows[i].copy())
                    i += 1
                cursor[e["id"]] = cursor.get(e["id"], 0) + len(e["tokens"])
        H.compare(got, ref, tol, "trace_run " + dname)


def test_weights_stored_in_32_bit_stay_so_in_bfloat16_mode(tmp_path_factory):
    """A folder whose tensors are all float32, run with --dtype bfloat16: matrices stay float32
    (their products run in float32), activations and the cache are bfloat16."""
    from infinicore_infer_amd.engine import Engine
    folder = H.make_model_dir(tmp_path_factory.getbasetemp(), "B", seed=4, dtype=torch.float32)
    requests = {"a": H.random_tokens(509, 70, 1), "b": H.random_tokens(509, 33, 2)}
    steps, max_tokens = H.trace_mixed(requests, sizes=(11, 2, 6), tail=4)
    engine = Engine.from_dir(folder, dtype=torch.bfloat16, max_tokens=max_tokens, page_size=16, max_requests=4)
    assert engine.model.layers[0].mixer.w_qkv.dtype == torch.float32
    assert engine.storage.kv(0)[0].dtype == torch.bfloat16
    ref = H.plain_logits(H.CONFIGS["B"][0], H.load_state_dict(folder), requests, True)
    H.compare(H.run_trace(engine, steps), ref, H.BF16_TOL, "float32 folder in bfloat16 mode")


def test_benchmark_shaped_layers(tmp_path_factory):
    """Two layers with the benchmark model's sizes (hidden 2304, 36 heads of 64, intermediate 5760,
    an odd vocabulary of 30001), bfloat16: a prompt in portions that span several attention tiles, then
    single tokens whose keys are split 16 ways, beside a second request; page size 64."""
    from infinicore_infer_amd.engine import Engine
    from infinicore_infer_amd.weights import write_random_model
    import os
    cfg = dict(model_type="minicpm", vocab_size=30001, hidden_size=2304, num_hidden_layers=2,
               num_attention_heads=36, num_key_value_heads=36, intermediate_size=5760,
               max_position_embeddings=1024, rms_norm_eps=1e-5, rope_theta=10000.0, scale_emb=12,
               dim_model_base=256, scale_depth=1.4, tie_word_embeddings=True, eos_token_id=2)
    folder = os.path.join(str(tmp_path_factory.getbasetemp()), "model_2b_shaped")
    write_random_model(folder, cfg, seed=9, std=0.02)
    sd = H.load_state_dict(folder)
    a, b = H.random_tokens(30001, 420, 1), H.random_tokens(30001, 70, 2)
    want_a, want_b = [0, 127, 128, 299, 300, 409] + list(range(410, 420)), [0, 69]
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": a[:300], "want": [0, 127, 128, 299]}], "end": []},
        {"step": 1, "entries": [{"id": "a", "tokens": a[300:410], "want": [0, 109]},
                                {"id": "b", "tokens": b[:69], "want": [0]}], "end": []},
    ]
    for i in range(410, 420):
        ents = [{"id": "a", "tokens": [a[i]], "want": [0]}]
        if i == 410:
            ents.append({"id": "b", "tokens": [b[69]], "want": [0]})
        steps.append({"step": len(steps), "entries": ents, "end": ["b"] if i == 410 else []})
    steps[-1]["end"] = ["a"]
    engine = Engine.from_dir(folder, dtype=torch.bfloat16, max_tokens=576, page_size=64, max_requests=2)
    got = H.run_trace(engine, steps)
    from plain_model import plain_forward, round_bf16
    ref_a = plain_forward(cfg, sd, a, rnd=round_bf16, rows=want_a)
    ref_b = plain_forward(cfg, sd, b, rnd=round_bf16, rows=want_b)
    ref = {"a": {p: ref_a[i] for i, p in enumerate(want_a)}, "b": {p: ref_b[i] for i, p in enumerate(want_b)}}
    assert sorted(got) == sorted([("a", p) for p in want_a] + [("b", p) for p in want_b])
    scale = float(max(ref_a.abs().max(), ref_b.abs().max()))
    for (rid, pos), row in got.items():
        err = float((row.double() - ref[rid][pos]).abs().max()) / scale
        assert err <= H.BF16_TOL, "request %s position %d differs by %.3g of the largest logit" % (rid, pos, err)
    assert engine.graph_steps + engine.graph_deferred >= 9 and engine.graph_replays >= 6


def test_a_shape_is_recorded_when_it_comes_back(tmp_path_factory):
    """While requests join and leave, most decode shapes (batch size, key-count bucket) are seen once: such a step runs
    eagerly.  A shape that comes back is recorded then and replayed afterwards.  All three ways give the same bits."""
    from infinicore_infer_amd.engine import Engine, StepEntry
    cfg = H.CONFIGS["A"][0]
    folder = H.make_model_dir(tmp_path_factory.getbasetemp(), "A")
    a = Engine.from_dir(folder, dtype=torch.bfloat16, max_tokens=512, page_size=16, max_requests=4)
    b = Engine.from_dir(folder, dtype=torch.bfloat16, max_tokens=512, page_size=16, max_requests=4, use_graphs=False)
    assert a.graph_after == 2
    ids = ["x", "y", "z"]
    for eng in (a, b):
        eng.step([StepEntry(r, H.random_tokens(cfg["vocab_size"], 5 + 3 * i, i), []) for i, r in enumerate(ids)])
    toks = H.random_tokens(cfg["vocab_size"], 40, 8)
    seen = []
    for i, n in enumerate([3, 2, 1, 3, 3, 2, 3, 1, 1]):          # batch sizes as requests pause and resume
        ents = [StepEntry(r, [toks[i + j]], [0]) for j, r in enumerate(ids[:n])]
        assert torch.equal(a.step(ents).clone(), b.step(ents).clone()), "step %d" % i
        seen.append((a.graph_deferred, a.graph_steps, a.graph_replays, len(a._graphs)))
    # sizes 3, 2, 1 first run eagerly; the second 3 records, the third replays; the second 2 records; ...
    assert seen[2] == (3, 0, 0, 0) and seen[3] == (3, 1, 0, 1) and seen[4] == (3, 2, 1, 1)
    assert seen[5] == (3, 3, 1, 2) and seen[6] == (3, 4, 2, 2) and seen[7] == (3, 5, 2, 3) and seen[8] == (3, 6, 3, 3)


@pytest.mark.parametrize("native", [True, False])
def test_recorded_steps_hold_a_bounded_amount_of_memory(tmp_path_factory, native):
    """Every batch size from 1 to 64 decodes once.  Recordings beyond ``max_graphs`` push out the least
    recently used one; a natively stepped model's recordings share one workspace sized for the largest
    batch, so the bytes they hold stay under a cap that does not depend on how many shapes were seen."""
    from infinicore_infer_amd.engine import Engine, StepEntry
    cfg = H.CONFIGS["C"][0]
    folder = H.make_model_dir(tmp_path_factory.getbasetemp(), "C")
    eng = Engine.from_dir(folder, dtype=torch.bfloat16, max_tokens=64 * 64, page_size=16, max_requests=64,
                          max_graphs=12, use_native=native, graph_after=1)
    ids = ["g%d" % i for i in range(64)]
    eng.step([StepEntry(r, H.random_tokens(cfg["vocab_size"], 3 + i % 9, i), []) for i, r in enumerate(ids)])
    sizes = []
    for n in range(1, 65):
        out = eng.step([StepEntry(r, [1 + i], [0]) for i, r in enumerate(ids[:n])])
        assert out.shape == (n, cfg["vocab_size"])
        sizes.append(eng.graph_bytes())
        assert len(eng._graphs) <= 12
    assert eng.graph_steps == 64 and eng.graphs_evicted == 64 - 12
    meta_bytes = 12 * 4 * (64 * (7 + cfg["max_position_embeddings"] // 16) + 64)
    if native:
        cap = eng.native.workspace_bytes_for_decode(64) + 64 * cfg["vocab_size"] * 4 + meta_bytes
        assert max(sizes) <= cap, (max(sizes), cap)
    else:
        # a workspace per recording: bounded by max_graphs times the largest one
        biggest = max(g.ctx.ws.bytes() + g.meta.numel() * 4 for g in eng._graphs.values())
        assert max(sizes) <= 12 * biggest
    assert sizes[-1] <= 1.05 * max(sizes[11:])            # no growth once the cap on recordings is reached
    # a recording that was pushed out is made again when its shape comes back, with the right result
    again = eng.step([StepEntry(r, [9], [0]) for r in ids[:2]]).clone()
    ref = Engine.from_dir(folder, dtype=torch.bfloat16, max_tokens=64 * 64, page_size=16, max_requests=64, use_graphs=False)
    ref.step([StepEntry(r, H.random_tokens(cfg["vocab_size"], 3 + i % 9, i), []) for i, r in enumerate(ids[:2])])
    for n in range(1, 65):
        if n <= 2:
            ref.step([StepEntry(r, [1 + i], [0]) for i, r in enumerate(ids[:min(n, 2)])])
        else:
            ref.step([StepEntry(r, [1 + i], [0]) for i, r in enumerate(ids[:2])])
    want = ref.step([StepEntry(r, [9], [0]) for r in ids[:2]])      # other batches, other kernels: equal to rounding
    assert float((again - want).abs().max()) <= H.BF16_TOL * float(want.abs().max())


@pytest.mark.parametrize("native", [True, False])
def test_prompt_portions_after_a_long_past_walk_their_keys_in_parts(tmp_path_factory, native):
    """A prompt of 2,000 tokens in portions of 512 beside a second request: from the fourth portion on the query
    tiles see 24 and more key tiles and there are few blocks, so each tile's walk over the keys is cut into parts
    that blocks of their own take (head size 64, grouped queries, page size 64, bfloat16).  Compared with the plain
    implementation at the first, the last and some other places of every portion."""
    import os
    from infinicore_infer_amd.engine import Engine
    from infinicore_infer_amd.kernels import ops
    from infinicore_infer_amd.weights import write_random_model
    from plain_model import plain_forward, round_bf16
    cfg = dict(model_type="minicpm", vocab_size=1009, hidden_size=256, num_hidden_layers=2, num_attention_heads=4,
               num_key_value_heads=2, intermediate_size=384, max_position_embeddings=2048, rms_norm_eps=1e-5,
               rope_theta=10000.0, scale_emb=4, dim_model_base=64, scale_depth=1.2, tie_word_embeddings=False, eos_token_id=2)
    folder = os.path.join(str(tmp_path_factory.getbasetemp()), "model_long_past")
    if not os.path.exists(os.path.join(folder, "config.json")):
        write_random_model(folder, cfg, seed=21, std=0.05)
    sd = H.load_state_dict(folder)
    a, b = H.random_tokens(1009, 2000, 5), H.random_tokens(1009, 700, 6)
    cuts_a = [0, 512, 1024, 1536, 1900, 2000]
    cuts_b = [0, 0, 300, 300, 700, 700]                    # b's portions ride along in the third and fifth step
    steps, want_a, want_b = [], [], []
    for i in range(5):
        ents = []
        n = cuts_a[i + 1] - cuts_a[i]
        w = sorted({0, 1, n // 2, n - 2, n - 1})
        ents.append({"id": "a", "tokens": a[cuts_a[i]:cuts_a[i + 1]], "want": w})
        want_a += [cuts_a[i] + j for j in w]
        nb = cuts_b[i + 1] - cuts_b[i]
        if nb:
            wb = [0, nb - 1]
            ents.append({"id": "b", "tokens": b[cuts_b[i]:cuts_b[i + 1]], "want": wb})
            want_b += [cuts_b[i] + j for j in wb]
        steps.append({"step": i, "entries": ents, "end": []})
    steps[-1]["end"] = ["a", "b"]
    engine = Engine.from_dir(folder, dtype=torch.bfloat16, max_tokens=2048 + 704, page_size=64, max_requests=2, use_native=native)
    assert (engine.native is not None) == native
    # the rule really cuts these steps: 4 and 3 tiles of the first request (and 4 of the second) with 4 heads
    assert ops.attention_prefill_parts(4, 4, 64, 2048, engine.cu_count)[0] == 4
    assert ops.attention_prefill_parts(3 + 4, 4, 64, 1900, engine.cu_count)[0] == 4
    got = H.run_trace(engine, steps)
    ref_a = plain_forward(cfg, sd, a, rnd=round_bf16, rows=want_a)
    ref_b = plain_forward(cfg, sd, b, rnd=round_bf16, rows=want_b)
    ref = {"a": {p: ref_a[i] for i, p in enumerate(want_a)}, "b": {p: ref_b[i] for i, p in enumerate(want_b)}}
    assert sorted(got) == sorted([("a", p) for p in want_a] + [("b", p) for p in want_b])
    scale = float(max(ref_a.abs().max(), ref_b.abs().max()))
    for (rid, pos), row in sorted(got.items()):
        err = float((row.double() - ref[rid][pos]).abs().max()) / scale
        assert err <= H.BF16_TOL, "request %s position %d differs by %.3g of the largest logit" % (rid, pos, err)
