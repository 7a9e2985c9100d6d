"""Each part alone against its plain function; greedy generation through the entry point and
the scheduler; and a toy architecture defined HERE (a mixer with state of its own, a windowed
attention layer, a layer that reads another layer's cache, a layer run twice) that is registered,
built and stepped without a change to the framework's files."""
import math

import pytest
import torch

import helpers as H
import plain_model as P

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


# ---------------------------------------------------------------------------
# a hand-made step context: one or more requests, identity page mapping
# ---------------------------------------------------------------------------
def _context(lens, page_size, n_kv_heads, head_dim, dtype, n_slots=1):
    """lens: list of (past, new).  Pages are laid out one request after the other."""
    from infinicore_infer_amd.engine.context import LayerCacheView, StepContext, Workspace
    ctx = StepContext()
    positions, token_req, slots, tables, dec, tiles = [], [], [], [], [], []
    page0, row0 = 0, 0
    maxb = max((p + n + page_size - 1) // page_size for p, n in lens)
    for r, (past, new) in enumerate(lens):
        nb = (past + new + page_size - 1) // page_size
        tables.append(list(range(page0, page0 + nb)) + [0] * (maxb - nb))
        for p in range(past, past + new):
            positions.append(p)
            token_req.append(r)
            slots.append((page0 + p // page_size) * page_size + p % page_size)
        if new == 1:
            dec.append(row0)
        else:
            for o in range(0, new, 128):
                tiles += [r, row0 + o, min(128, new - o), past + o]
        page0 += nb
        row0 += new
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
    ctx.T, ctx.R, ctx.page_size, ctx.ws = row0, len(lens), page_size, Workspace(DEV)
    ctx.positions, ctx.token_req = i32(positions), i32(token_req)
    ctx.decode_rows, ctx.n_decode_rows = i32(dec), len(dec)
    ctx.decode_rows_identity = len(dec) == row0
    ctx.prefill_tiles, ctx.n_prefill_tiles = i32(tiles).view(-1, 4), len(tiles) // 4
    ctx.max_position = max(positions)
    ctx.max_context = max(positions) + 1
    views = []
    for _ in range(n_slots):
        k = torch.zeros(page0, n_kv_heads, page_size, head_dim, dtype=dtype, device=DEV)
        views.append(LayerCacheView(k=k, v=torch.zeros_like(k), slots=i32(slots),
                                    block_tables=i32(tables).view(len(lens), maxb)))
    return ctx, views


def _rel(got, want):
    got, want = got.double().cpu(), want.double().cpu()
    return float((got - want).abs().max()) / float(want.abs().max())


DT = [(torch.float32, 2e-5), (torch.bfloat16, 2e-2)]


@pytest.mark.parametrize("dtype,tol", DT)
def test_norm_part(dtype, tol):
    from infinicore_infer_amd.parts import Runtime, build_part
    from infinicore_infer_amd.config import PartSpec
    rt = Runtime(dtype, DEV)
    norm = build_part("norm", PartSpec("rmsnorm", "n.", {"size": 200, "eps": 1e-6}), rt)
    assert list(norm.weight_specs()) == ["n.weight"]
    w = 1 + 0.2 * torch.randn(200)
    norm.load_weights({"n.weight": w.to(DEV)})
    x = torch.randn(9, 200)
    y = torch.randn(9, 200).to(dtype)
    out = torch.empty(9, 200, dtype=dtype, device=DEV)
    norm.forward(x.to(DEV), out)
    assert _rel(out, P.plain_rmsnorm(x, w, 1e-6)) < tol
    xd = x.to(DEV).clone()
    norm.forward_add(xd, y.to(DEV), 0.5, out)
    assert _rel(out, P.plain_rmsnorm(x.double() + 0.5 * y.double(), w, 1e-6)) < tol


@pytest.mark.parametrize("dtype,tol", DT)
def test_feed_forward_part(dtype, tol):
    from infinicore_infer_amd.parts import Runtime, build_part
    from infinicore_infer_amd.config import PartSpec
    rt = Runtime(dtype, DEV)
    ffn = build_part("feed_forward", PartSpec("swiglu", "m.", {"hidden_size": 72, "intermediate_size": 200}), rt)
    w = {"m.gate_proj.weight": torch.randn(200, 72) * 0.1, "m.up_proj.weight": torch.randn(200, 72) * 0.1,
         "m.down_proj.weight": torch.randn(72, 200) * 0.1}
    w = {k: v.to(dtype) for k, v in w.items()}
    assert set(ffn.weight_specs()) == set(w)
    ffn.load_weights({k: v.to(DEV) for k, v in w.items()})
    ctx, _ = _context([(0, 11)], 16, 1, 16, dtype)
    h = torch.randn(11, 72).to(dtype)
    rnd = P.round_bf16 if dtype == torch.bfloat16 else (lambda t: t)
    act = rnd(P.plain_swiglu(rnd(P.plain_linear(h, w["m.gate_proj.weight"])), rnd(P.plain_linear(h, w["m.up_proj.weight"]))))
    want = P.plain_linear(act, w["m.down_proj.weight"])
    assert _rel(ffn.forward(h.to(DEV), ctx), want) < tol


@pytest.mark.parametrize("dtype,tol", DT)
@pytest.mark.parametrize("nh,nkvh,dh,window,scaling", [(4, 2, 16, None, None), (6, 2, 64, None, "long"),
                                                        (3, 3, 32, 20, None), (2, 1, 128, None, "short")])
def test_attention_and_rotary_parts(dtype, tol, nh, nkvh, dh, window, scaling):
    """The attention mixer (projection, rotary part, cache write, attention kernels, output
    projection) on a prompt portion with a past, and on single tokens, against the plain
    functions on the reference's permuted weights."""
    from infinicore_infer_amd.parts import Runtime, build_part
    from infinicore_infer_amd.config import PartSpec
    rt = Runtime(dtype, DEV)
    d, max_pos = 88, 256
    sc = None
    if scaling:
        sc = dict(type="longrope", original_max_position_embeddings=64 if scaling == "long" else 512,
                  short_factor=[1 + 0.1 * i for i in range(dh // 2)], long_factor=[2 + 0.1 * i for i in range(dh // 2)])
    rot = PartSpec("rotary", "", {"head_dim": dh, "theta": 5000.0, "max_positions": max_pos, "scaling": sc})
    att = build_part("mixer", PartSpec("attention", "a.", {
        "hidden_size": d, "num_heads": nh, "num_kv_heads": nkvh, "head_dim": dh,
        "softmax_scale": 1 / math.sqrt(dh), "window": window, "position_encoding": rot}), rt)
    g = torch.Generator().manual_seed(dh)
    w = {"a.q_proj.weight": torch.randn(nh * dh, d, generator=g) * 0.2, "a.k_proj.weight": torch.randn(nkvh * dh, d, generator=g) * 0.2,
         "a.v_proj.weight": torch.randn(nkvh * dh, d, generator=g) * 0.2, "a.o_proj.weight": torch.randn(d, nh * dh, generator=g) * 0.2}
    w = {k: v.to(dtype) for k, v in w.items()}
    att.load_weights({k: v.to(DEV) for k, v in w.items()})
    need = att.cache_need()
    assert (need.kind, need.n_kv_heads, need.head_dim, need.window) == ("kv", nkvh, dh, window)

    total, cut = 150, 97
    h = torch.randn(total, d, generator=g).to(dtype)
    rnd = P.round_bf16 if dtype == torch.bfloat16 else (lambda t: t)
    cfg = {"rope_scaling": sc, "max_position_embeddings": max_pos}
    factors, mag = P.plain_longrope(cfg)
    sin, cos = P.plain_rope_tables(dh, 5000.0, total, factors, mag)
    q = rnd(P.plain_linear(h, P.permute_rows_to_adjacent_pairs(w["a.q_proj.weight"].double(), nh, dh))).reshape(total, nh, dh)
    k = rnd(P.plain_linear(h, P.permute_rows_to_adjacent_pairs(w["a.k_proj.weight"].double(), nkvh, dh))).reshape(total, nkvh, dh)
    v = rnd(P.plain_linear(h, w["a.v_proj.weight"])).reshape(total, nkvh, dh)
    q = rnd(P.plain_rope_adjacent(q, range(total), sin, cos))
    k = rnd(P.plain_rope_adjacent(k, range(total), sin, cos))
    a = rnd(P.plain_attention(q, k, v, 1 / math.sqrt(dh), 0, window)).reshape(total, nh * dh)
    want = P.plain_linear(a, w["a.o_proj.weight"])

    # one cache for the whole test: first portion, second portion with a past, then single tokens
    ctx_all, views = _context([(0, total)], 16, nkvh, dh, dtype)
    view = views[0]
    from infinicore_infer_amd.engine.context import LayerCacheView
    got = torch.empty(total, d, dtype=dtype)
    pieces = [(0, cut), (cut, total - 3)] + [(i, i + 1) for i in range(total - 3, total)]
    for a0, a1 in pieces:
        ctx, _ = _context([(a0, a1 - a0)], 16, nkvh, dh, dtype)
        cv = LayerCacheView(k=view.k, v=view.v, slots=view.slots[a0:a1].contiguous(),
                            block_tables=view.block_tables)
        got[a0:a1] = att.forward(h[a0:a1].to(DEV), ctx, cv).cpu()
    assert _rel(got, want) < tol


def test_embedding_and_head_parts():
    from infinicore_infer_amd.parts import Runtime, build_part
    from infinicore_infer_amd.config import PartSpec
    rt = Runtime(torch.bfloat16, DEV)
    emb = build_part("embedding", PartSpec("embedding", "e.", {"vocab_size": 77, "hidden_size": 40, "scale": 3.0}), rt)
    head = build_part("head", PartSpec("lm_head", "h.", {"vocab_size": 77, "hidden_size": 40, "logit_scale": 0.5,
                                                         "fallback_name": "e."}), rt)
    norm = build_part("norm", PartSpec("rmsnorm", "n.", {"size": 40, "eps": 1e-5}), rt)
    assert head.weight_specs()["h.weight"].fallback == "e.weight"
    table = torch.randn(77, 40).to(torch.bfloat16)
    nw = 1 + 0.1 * torch.randn(40)
    emb.load_weights({"e.weight": table.to(DEV)})
    head.load_weights({"h.weight": table.to(DEV)})
    norm.load_weights({"n.weight": nw.to(DEV)})
    toks = [5, 76, 0, 5]
    x = torch.empty(4, 40, device=DEV)
    emb.forward(torch.tensor(toks, dtype=torch.int32, device=DEV), x)
    assert _rel(x, P.plain_embedding(table, toks, 3.0)) < 1e-6
    ctx, _ = _context([(0, 4)], 16, 1, 16, torch.bfloat16)
    rows = torch.tensor([3, 1], dtype=torch.int32, device=DEV)
    logits = head.forward(x, rows, norm, ctx)
    hn = P.round_bf16(P.plain_rmsnorm(x.cpu()[[3, 1]], nw, 1e-5) * 0.5)
    assert logits.dtype == torch.float32 and _rel(logits, P.plain_linear(hn, table)) < 2e-3


def test_weights_drawn_on_the_device_are_the_folder_written_on_the_cpu(tmp_path_factory):
    """Random-weights mode both ways: a folder written on the CPU and loaded, and weights drawn straight into a
    model on the GPU.  One seed, one model: every tensor is equal bit for bit, and so are the logits."""
    from infinicore_infer_amd.config import config_from_dict
    from infinicore_infer_amd.engine import Engine, StepEntry
    from infinicore_infer_amd.parts import Runtime, build_model
    from infinicore_infer_amd.weights import init_random_weights, standard_normal, write_random_model
    z = standard_normal(5, "model.embed_tokens.weight", 300001, device=DEV)
    assert torch.equal(z.cpu(), standard_normal(5, "model.embed_tokens.weight", 300001))
    for name, cfg, init in (("A", H.TINY_A, H.TINY_A_INIT), ("B", H.TINY_B, H.TINY_B_INIT)):
        folder = write_random_model(str(tmp_path_factory.mktemp("drawn_" + name)), cfg, seed=21, **init)
        loaded = Engine.from_dir(folder, dtype=torch.bfloat16, max_tokens=64)
        model = build_model(config_from_dict(cfg).model_spec(), Runtime(torch.bfloat16, DEV))
        init_random_weights(model, seed=21, tie=cfg.get("tie_word_embeddings", True), **init)
        drawn = Engine(model, max_tokens=64)
        la, lb = loaded.model.layers[-1], drawn.model.layers[-1]
        for x, y in ((loaded.model.embedding.table, drawn.model.embedding.table), (loaded.model.head.weight, drawn.model.head.weight),
                     (la.mixer.w_qkv, lb.mixer.w_qkv), (la.mixer.w_o, lb.mixer.w_o), (la.feed_forward.w_gate_up, lb.feed_forward.w_gate_up),
                     (la.feed_forward.w_down, lb.feed_forward.w_down), (la.feed_forward_norm.weight, lb.feed_forward_norm.weight),
                     (loaded.model.final_norm.weight, drawn.model.final_norm.weight)):
            assert x.dtype == y.dtype and torch.equal(x, y)
        toks = [3, 1, 4, 1, 5, 9, 2, 6]
        a = loaded.step([StepEntry("r", toks, list(range(len(toks))))])
        b = drawn.step([StepEntry("r", toks, list(range(len(toks))))])
        assert torch.equal(a, b)


# ---------------------------------------------------------------------------
# generation through the entry point and the scheduler
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("name", ["A", "B"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_greedy_generation_through_the_entry_point(tmp_path_factory, name, dtype):
    from infinicore_infer_amd.minicpm import MiniCPMForCausalLM
    folder = H.make_model_dir(tmp_path_factory.getbasetemp(), name, seed=7)
    cfg = H.CONFIGS[name][0]
    sd = H.load_state_dict(folder)
    prompt = H.random_tokens(cfg["vocab_size"], 11, 8)
    rnd = P.round_bf16 if dtype == torch.bfloat16 else None
    want = P.plain_generate(dict(cfg, eos_token_id=[]), sd, prompt, 8, rnd=rnd)
    model = MiniCPMForCausalLM(folder, DEV, 1, dtype=dtype, cache_tokens=256, page_size=16)
    model.eos_token_id = []
    out, _ = model.generate(prompt, 8)
    assert model.last_output_tokens == want
    # the same through the scheduler, three prompts at once, with so few pages that one is preempted
    prompts = [prompt, prompt[:5], prompt[3:]]
    wants = [P.plain_generate(dict(cfg, eos_token_id=[]), sd, p, 8, rnd=rnd) for p in prompts]
    model2 = MiniCPMForCausalLM(folder, DEV, 1, dtype=dtype, cache_tokens=48, page_size=16)
    model2.eos_token_id = []
    assert model2.generate_batch(prompts, 8, max_batch_tokens=16, chunk_size=6) == wants
    assert model2.engine.cache.free_pages(0) == 3
    ppl = model.perplexity([prompt, prompt[2:]], batch_size=2)
    logits = [P.plain_forward(cfg, sd, p[:-1], rnd=rnd) for p in (prompt, prompt[2:])]
    nll = sum(-float(torch.log_softmax(l, -1)[torch.arange(len(p) - 1), torch.tensor(p[1:])].sum())
              for l, p in zip(logits, (prompt, prompt[2:])))
    assert ppl == pytest.approx(math.exp(nll / (len(prompt) - 1 + len(prompt) - 3)), rel=2e-2 if rnd else 1e-4)


def test_temperature_sampling_is_reproducible(tmp_path_factory):
    from infinicore_infer_amd.minicpm import MiniCPMForCausalLM
    folder = H.make_model_dir(tmp_path_factory.getbasetemp(), "B", seed=7)
    model = MiniCPMForCausalLM(folder, DEV, 1, dtype=torch.float32, cache_tokens=256, page_size=16)
    model.eos_token_id = []
    prompts = [H.random_tokens(509, 9, 1), H.random_tokens(509, 4, 2)]
    a = model.generate_batch(prompts, 12, topp_=0.9, topk_=40, temperature_=1.5, seed=3)
    b = model.generate_batch(prompts, 12, topp_=0.9, topk_=40, temperature_=1.5, seed=3)
    c = model.generate_batch(prompts, 12, topp_=0.9, topk_=40, temperature_=1.5, seed=4)
    assert a == b and a != c


# ---------------------------------------------------------------------------
# a toy architecture, defined and registered here
# ---------------------------------------------------------------------------
def _register_toy():
    from infinicore_infer_amd.config import ExecEntry, LayerSpec, ModelSpec, PartSpec, register_architecture
    from infinicore_infer_amd.parts import CacheNeed, Mixer, register_part
    from infinicore_infer_amd.weights import WeightSpec

    @register_part("mixer", "toy_running_mean")
    class RunningMean(Mixer):
        """y_t = gain * mean(h_0..h_t): needs a running sum and a count per request."""

        def __init__(self, name, runtime, hidden_size):
            super().__init__(name, runtime)
            self.d = hidden_size
            self.gain = None

        def cache_need(self):
            return CacheNeed("state", state_shape=(self.d + 1,), state_dtype=torch.float32)

        def weight_specs(self):
            return {self.name + "gain": WeightSpec((self.d,), "vector")}

        def load_weights(self, tensors):
            self.gain = tensors[self.name + "gain"]

        def forward(self, h, ctx, cache):
            y = ctx.ws.buffer("toy_out", tuple(h.shape), self.runtime.dtype)
            for r in range(ctx.R):
                a, b = ctx.req_start[r], ctx.req_start[r + 1]
                st = cache.state[ctx.host_state_slots[r]]
                cs = torch.cumsum(h[a:b].float(), 0) + st[:-1]
                n = st[-1] + torch.arange(1, b - a + 1, device=h.device)
                y[a:b] = (cs / n[:, None] * self.gain).to(y.dtype)
                st[:-1] = cs[-1]
                st[-1] = n[-1]
            return y

    class ToyConfig:
        def __init__(self, cfg):
            self.cfg = cfg

        @classmethod
        def from_dict(cls, cfg, **kw):
            return cls(cfg)

        def model_spec(self):
            c = self.cfg
            d, nh, nkvh, dh = c["hidden"], c["heads"], c["kv_heads"], c["head_dim"]
            rot = PartSpec("rotary", "", {"head_dim": dh, "theta": 1000.0, "max_positions": c["max_pos"]})

            def norm(p):
                return PartSpec("rmsnorm", p, {"size": d, "eps": 1e-5})

            def ffn(p):
                return PartSpec("swiglu", p, {"hidden_size": d, "intermediate_size": c["inter"]})

            def attn(p, **kw):
                return PartSpec("attention", p, dict({"hidden_size": d, "num_heads": nh, "num_kv_heads": nkvh,
                                                      "head_dim": dh, "softmax_scale": dh ** -0.5,
                                                      "position_encoding": rot}, **kw))
            block = lambda p: PartSpec("prenorm_residual", p, {"residual_scale": 0.8})
            layers = [
                LayerSpec(block("l0."), attn("l0.att.", window=c["window"]), norm("l0.n1."), ffn("l0.ffn."), norm("l0.n2.")),
                LayerSpec(block("l1."), PartSpec("toy_running_mean", "l1.mix.", {"hidden_size": d}), norm("l1.n1."),
                          ffn("l1.ffn."), norm("l1.n2.")),
                LayerSpec(block("l2."), attn("l2.att.", window=c["window"], shared_kv=True), norm("l2.n1."),
                          ffn("l2.ffn."), norm("l2.n2.")),
                LayerSpec(block("l3."), attn("l3.att."), norm("l3.n1."), ffn("l3.ffn."), norm("l3.n2.")),
            ]
            schedule = [ExecEntry(0, 0, True), ExecEntry(1, 1, True), ExecEntry(2, 0, False),
                        ExecEntry(3, 2, True), ExecEntry(1, 3, True)]       # layer 1 runs twice, each run with its own state
            return ModelSpec("toy", c["vocab"], d, c["max_pos"],
                             PartSpec("embedding", "emb.", {"vocab_size": c["vocab"], "hidden_size": d, "scale": 2.0}),
                             layers, schedule, norm("final."),
                             PartSpec("lm_head", "head.", {"vocab_size": c["vocab"], "hidden_size": d, "logit_scale": 1.0,
                                                           "fallback_name": "emb."}))

    register_architecture(["toy-test-arch"], ToyConfig)


def _toy_plain(model, cfg, tokens):
    """The toy model in plain float64, whole sequence."""
    T = len(tokens)
    d, nh, nkvh, dh, win = cfg["hidden"], cfg["heads"], cfg["kv_heads"], cfg["head_dim"], cfg["window"]
    half = dh // 2
    cpu = lambda t: t.detach().cpu().double()
    sin, cos = P.plain_rope_tables(dh, 1000.0, T)

    def rope(x):
        s, c = sin[:T, None, :], cos[:T, None, :]
        return torch.cat([x[..., :half] * c - x[..., half:] * s, x[..., :half] * s + x[..., half:] * c], -1)

    x = P.plain_embedding(cpu(model.embedding.table), tokens, 2.0)
    kv = {}
    for e in model.schedule:
        blk = model.layers[e.layer]
        h = P.plain_rmsnorm(x, cpu(blk.mixer_norm.weight), 1e-5)
        m = blk.mixer
        if hasattr(m, "gain"):
            y = torch.cumsum(h, 0) / torch.arange(1, T + 1)[:, None] * cpu(m.gain)
        else:
            qkv = P.plain_linear(h, cpu(m.w_qkv))
            q = rope(qkv[:, :nh * dh].reshape(T, nh, dh))
            if e.writes_cache:
                k = rope(qkv[:, nh * dh:(nh + nkvh) * dh].reshape(T, nkvh, dh))
                v = qkv[:, (nh + nkvh) * dh:].reshape(T, nkvh, dh)
                kv[e.cache] = (k, v)
            k, v = kv[e.cache]
            a = P.plain_attention(q, k, v, dh ** -0.5, 0, m.window or None).reshape(T, nh * dh)
            y = P.plain_linear(a, cpu(m.w_o))
        x = x + 0.8 * y
        h = P.plain_rmsnorm(x, cpu(blk.feed_forward_norm.weight), 1e-5)
        gu = P.plain_linear(h, cpu(blk.feed_forward.w_gate_up))
        di = gu.shape[1] // 2
        x = x + 0.8 * P.plain_linear(P.plain_swiglu(gu[:, :di], gu[:, di:]), cpu(blk.feed_forward.w_down))
    return P.plain_linear(P.plain_rmsnorm(x, cpu(model.final_norm.weight), 1e-5), cpu(model.head.weight))


def test_toy_architecture_with_a_stateful_mixer(tmp_path_factory):
    from infinicore_infer_amd.config import config_from_dict
    from infinicore_infer_amd.engine import Engine
    from infinicore_infer_amd.parts import Runtime, build_model
    from infinicore_infer_amd.weights import init_random_weights
    _register_toy()
    cfg = {"model_type": "toy-test-arch", "vocab": 97, "hidden": 48, "heads": 4, "kv_heads": 2, "head_dim": 16,
           "inter": 80, "window": 24, "max_pos": 256}
    model = build_model(config_from_dict(cfg).model_spec(), Runtime(torch.float32, DEV))
    init_random_weights(model, seed=11, std=0.15, norm_std=0.1, tie=True)
    needs = model.cache_needs()
    assert [n.kind for n in needs] == ["kv", "state", "kv", "state"]
    assert needs[0].window == 24 and needs[2].window is None
    requests = {"t%d" % i: H.random_tokens(97, n, 40 + i) for i, n in enumerate([70, 33, 120, 9])}
    ref = {rid: _toy_plain(model, cfg, toks) for rid, toks in requests.items()}
    for maker in (H.trace_whole, H.trace_chunks, H.trace_mixed):
        steps, max_tokens = maker(requests)
        eng = Engine(model, max_tokens=max_tokens, page_size=16, max_requests=4)
        assert len(eng.groups) == 2 and {g.kind for g in eng.groups} == {"full", "window"}
        got = H.run_trace(eng, steps)
        H.compare(got, ref, 1e-4, "toy %s" % maker.__name__)
        eng.cache.check_invariants()
        assert all(eng.cache.free_pages(g) == eng.num_pages for g in range(2))
    # the window group really gives pages back while a long request runs
    eng = Engine(model, max_tokens=128, page_size=16, max_requests=2)
    from infinicore_infer_amd.engine import StepEntry
    eng.step([StepEntry("w", requests["t2"][:100], [])])
    wg = [i for i, g in enumerate(eng.groups) if g.kind == "window"][0]
    assert eng.cache.free_pages(wg) > eng.cache.free_pages(1 - wg)


# ---------------------------------------------------------------------------
# a second toy architecture: a feed-forward with routing and another position encoding
# ---------------------------------------------------------------------------
def _register_toy_routed():
    from infinicore_infer_amd.config import LayerSpec, ModelSpec, PartSpec, default_schedule, register_architecture
    from infinicore_infer_amd.parts import FeedForward, PositionEncoding, register_part
    from infinicore_infer_amd.parts.rotary import NoPositionEncoding
    from infinicore_infer_amd.weights import WeightSpec

    @register_part("feed_forward", "toy_top1_experts")
    class Top1Experts(FeedForward):
        """Router logits in float32, the best expert per token, experts = up, GELU, down."""

        def __init__(self, name, runtime, hidden_size, inner_size, num_experts):
            super().__init__(name, runtime)
            self.d, self.di, self.ne = hidden_size, inner_size, num_experts

        def weight_specs(self):
            n = self.name
            s = {n + "router.weight": WeightSpec((self.ne, self.d))}
            for i in range(self.ne):
                s[n + "experts.%d.up.weight" % i] = WeightSpec((self.di, self.d))
                s[n + "experts.%d.down.weight" % i] = WeightSpec((self.d, self.di))
            return s

        def load_weights(self, tensors):
            n = self.name
            self.router = tensors[n + "router.weight"]
            self.up = [tensors[n + "experts.%d.up.weight" % i] for i in range(self.ne)]
            self.down = [tensors[n + "experts.%d.down.weight" % i] for i in range(self.ne)]

        def forward(self, h, ctx):
            choice = (h.float() @ self.router.float().t()).argmax(-1)
            y = ctx.ws.buffer("toy_ffn_out", tuple(h.shape), self.runtime.dtype)
            for i in range(self.ne):
                rows = (choice == i).nonzero().flatten()
                if rows.numel():
                    a = torch.nn.functional.gelu(h[rows] @ self.up[i].t())
                    y[rows] = a @ self.down[i].t()
            return y

    @register_part("position_encoding", "toy_adjacent_pairs")
    class AdjacentPairs(PositionEncoding):
        """Rotates pairs (2j, 2j + 1) of q and k by pos * base^-j, then stores k and v as they are."""

        def __init__(self, name, runtime, head_dim, base):
            super().__init__(name, runtime)
            self.dh, self.base = head_dim, float(base)
            self.store = NoPositionEncoding(name, runtime)

        def rotate_and_store(self, qkv, ctx, cache, n_heads, n_kv_heads, head_dim):
            T = qkv.shape[0]
            j = torch.arange(head_dim // 2, device=qkv.device, dtype=torch.float32)
            ang = ctx.positions.float()[:, None] * self.base ** (-j)[None, :]
            c, s = ang.cos()[:, None, :], ang.sin()[:, None, :]
            x = qkv[:, :(n_heads + n_kv_heads) * head_dim].reshape(T, n_heads + n_kv_heads, head_dim // 2, 2).float()
            a, b = x[..., 0], x[..., 1]
            rot = torch.stack([a * c - b * s, a * s + b * c], -1).reshape(T, -1)
            qkv[:, :(n_heads + n_kv_heads) * head_dim] = rot.to(qkv.dtype)
            self.store.rotate_and_store(qkv, ctx, cache, n_heads, n_kv_heads, head_dim)

    class RoutedConfig:
        def __init__(self, cfg):
            self.cfg = cfg

        @classmethod
        def from_dict(cls, cfg, **kw):
            return cls(cfg)

        def model_spec(self):
            c = self.cfg
            d, nh, dh = c["hidden"], c["heads"], c["head_dim"]
            pe = PartSpec("toy_adjacent_pairs", "", {"head_dim": dh, "base": c["base"]})
            norm = lambda p: PartSpec("rmsnorm", p, {"size": d, "eps": 1e-6})
            layers = []
            for i in range(c["layers"]):
                p = "blocks.%d." % i
                ffn = PartSpec("toy_top1_experts", p + "moe.", {"hidden_size": d, "inner_size": c["inner"], "num_experts": c["experts"]}) \
                    if i % 2 == 0 else PartSpec("swiglu", p + "mlp.", {"hidden_size": d, "intermediate_size": c["inner"]})
                att = PartSpec("attention", p + "att.", {"hidden_size": d, "num_heads": nh, "num_kv_heads": nh, "head_dim": dh,
                                                         "softmax_scale": dh ** -0.5, "position_encoding": pe})
                layers.append(LayerSpec(PartSpec("prenorm_residual", p, {"residual_scale": 1.0}), att, norm(p + "n1."),
                                        ffn, norm(p + "n2.")))
            return ModelSpec("toy-routed", c["vocab"], d, c["max_pos"],
                             PartSpec("embedding", "emb.", {"vocab_size": c["vocab"], "hidden_size": d, "scale": 1.0}),
                             layers, default_schedule(len(layers)), norm("final."),
                             PartSpec("lm_head", "head.", {"vocab_size": c["vocab"], "hidden_size": d, "logit_scale": 1.0}))

    register_architecture(["toy-routed-arch"], RoutedConfig)


def _toy_routed_plain(model, cfg, tokens):
    T, nh, dh = len(tokens), cfg["heads"], cfg["head_dim"]
    cpu = lambda t: t.detach().cpu().double()
    j = torch.arange(dh // 2, dtype=torch.float64)
    ang = torch.arange(T, dtype=torch.float64)[:, None] * cfg["base"] ** (-j)[None, :]
    c, s = ang.cos()[:, None, :], ang.sin()[:, None, :]

    def rot(x):                                     # [T, heads, dh], adjacent pairs
        a, b = x[..., 0::2], x[..., 1::2]
        return torch.stack([a * c - b * s, a * s + b * c], -1).reshape(x.shape)

    x = P.plain_embedding(cpu(model.embedding.table), tokens, 1.0)
    for blk in model.layers:
        h = P.plain_rmsnorm(x, cpu(blk.mixer_norm.weight), 1e-6)
        qkv = P.plain_linear(h, cpu(blk.mixer.w_qkv)).reshape(T, 3 * nh, dh)
        q, k, v = rot(qkv[:, :nh]), rot(qkv[:, nh:2 * nh]), qkv[:, 2 * nh:]
        a = P.plain_attention(q, k, v, dh ** -0.5, 0, None).reshape(T, nh * dh)
        x = x + P.plain_linear(a, cpu(blk.mixer.w_o))
        h = P.plain_rmsnorm(x, cpu(blk.feed_forward_norm.weight), 1e-6)
        f = blk.feed_forward
        if hasattr(f, "router"):
            choice = P.plain_linear(h, cpu(f.router)).argmax(-1)
            y = torch.zeros_like(h)
            for t in range(T):
                i = int(choice[t])
                y[t] = P.plain_linear(torch.nn.functional.gelu(P.plain_linear(h[t:t + 1], cpu(f.up[i]))), cpu(f.down[i]))[0]
        else:
            gu = P.plain_linear(h, cpu(f.w_gate_up))
            di = gu.shape[1] // 2
            y = P.plain_linear(P.plain_swiglu(gu[:, :di], gu[:, di:]), cpu(f.w_down))
        x = x + y
    return P.plain_linear(P.plain_rmsnorm(x, cpu(model.final_norm.weight), 1e-6), cpu(model.head.weight))


def test_toy_architecture_with_routed_experts_and_another_position_encoding():
    """A feed-forward with routing and a position encoding of its own, both defined here, chosen
    layer by layer beside the package's parts, registered, built and stepped through the engine."""
    from infinicore_infer_amd.config import config_from_dict
    from infinicore_infer_amd.engine import Engine
    from infinicore_infer_amd.parts import Runtime, build_model
    from infinicore_infer_amd.weights import init_random_weights
    _register_toy_routed()
    cfg = {"model_type": "toy-routed-arch", "vocab": 61, "hidden": 40, "heads": 5, "head_dim": 16, "inner": 56,
           "experts": 3, "layers": 3, "base": 50.0, "max_pos": 128}
    model = build_model(config_from_dict(cfg).model_spec(), Runtime(torch.float32, DEV))
    init_random_weights(model, seed=5, std=0.2, norm_std=0.1, tie=False)
    requests = {"m%d" % i: H.random_tokens(61, n, 60 + i) for i, n in enumerate([50, 17, 90])}
    ref = {rid: _toy_routed_plain(model, cfg, toks) for rid, toks in requests.items()}
    used = set()
    for blk in model.layers:
        if hasattr(blk.feed_forward, "router"):
            used.add(type(blk.feed_forward).__name__)
    assert used == {"Top1Experts"}
    for maker in (H.trace_whole, H.trace_chunks, H.trace_mixed):
        steps, max_tokens = maker(requests)
        eng = Engine(model, max_tokens=max_tokens, page_size=16, max_requests=4)
        assert not eng.use_graphs                      # parts that do not declare graph_safe keep the engine eager
        got = H.run_trace(eng, steps)
        H.compare(got, ref, 2e-4, "toy routed %s" % maker.__name__)
        eng.cache.check_invariants()


# ---------------------------------------------------------------------------
# a third toy architecture: a mixer that caches ONE latent vector per token in pages (one plane,
# no keys and values, no heads) and carries a running state per request beside it
# ---------------------------------------------------------------------------
def _register_toy_latent():
    from infinicore_infer_amd.config import LayerSpec, ModelSpec, PartSpec, default_schedule, register_architecture
    from infinicore_infer_amd.parts import CacheNeed, Mixer, register_part
    from infinicore_infer_amd.weights import WeightSpec

    @register_part("mixer", "toy_latent_memory")
    class LatentMemory(Mixer):
        """c_t = W_down h_t is cached; y_t = W_up (sum_s softmax_s(c_t . c_s / sqrt(L)) c_s + mean_{s <= t} c_s),
        s over the tokens up to t.  The softmax walks the paged latents, the mean comes from a running
        sum and count kept as the request's state."""

        def __init__(self, name, runtime, hidden_size, latent_size):
            super().__init__(name, runtime)
            self.d, self.L = hidden_size, latent_size

        def cache_need(self):
            return CacheNeed("kv+state", n_kv_heads=1, head_dim=self.L, planes=1, state_shape=(self.L + 1,),
                             state_dtype=torch.float32)

        def weight_specs(self):
            return {self.name + "down.weight": WeightSpec((self.L, self.d)), self.name + "up.weight": WeightSpec((self.d, self.L))}

        def load_weights(self, tensors):
            self.w_down, self.w_up = tensors[self.name + "down.weight"], tensors[self.name + "up.weight"]

        def forward(self, h, ctx, cache):
            assert len(cache.planes) == 1 and cache.v is None and cache.state is not None
            ps = ctx.page_size
            c = (h @ self.w_down.t()).float()
            latents = cache.planes[0].view(-1, self.L)               # [pages * page_size, L]: one row per token slot
            if cache.writes:
                latents[cache.slots.long()] = c.to(latents.dtype)
            y = ctx.ws.buffer("toy_latent_out", tuple(h.shape), self.runtime.dtype)
            for r in range(ctx.R):
                a, b, p0 = ctx.req_start[r], ctx.req_start[r + 1], ctx.req_pos[r]
                pos = torch.arange(p0 + b - a, device=h.device)
                mem = latents[cache.block_tables[r].long()[pos // ps] * ps + pos % ps].float()       # every latent so far
                scores = c[a:b] @ mem.t() / self.L ** 0.5
                scores = scores.masked_fill(pos[None, :] > pos[p0:, None], float("-inf"))
                st = cache.state[ctx.host_state_slots[r]]
                run = torch.cumsum(c[a:b], 0) + st[:-1]
                n = st[-1] + torch.arange(1, b - a + 1, device=h.device)
                y[a:b] = ((torch.softmax(scores, -1) @ mem + run / n[:, None]) @ self.w_up.float().t()).to(y.dtype)
                st[:-1] = run[-1]
                st[-1] = n[-1]
            return y

    class LatentConfig:
        def __init__(self, cfg):
            self.cfg = cfg

        @classmethod
        def from_dict(cls, cfg, **kw):
            return cls(cfg)

        def model_spec(self):
            c = self.cfg
            d, nh, dh = c["hidden"], c["heads"], c["head_dim"]
            rot = PartSpec("rotary", "", {"head_dim": dh, "theta": 500.0, "max_positions": c["max_pos"]})
            norm = lambda p: PartSpec("rmsnorm", p, {"size": d, "eps": 1e-5})
            layers = []
            for i in range(3):
                p = "layers.%d." % i
                mixer = PartSpec("toy_latent_memory", p + "mem.", {"hidden_size": d, "latent_size": c["latent"]}) if i != 1 else \
                    PartSpec("attention", p + "att.", {"hidden_size": d, "num_heads": nh, "num_kv_heads": 1, "head_dim": dh,
                                                       "softmax_scale": dh ** -0.5, "position_encoding": rot})
                layers.append(LayerSpec(PartSpec("prenorm_residual", p, {"residual_scale": 0.7}), mixer, norm(p + "n1."),
                                        PartSpec("swiglu", p + "mlp.", {"hidden_size": d, "intermediate_size": c["inner"]}),
                                        norm(p + "n2.")))
            return ModelSpec("toy-latent", c["vocab"], d, c["max_pos"],
                             PartSpec("embedding", "emb.", {"vocab_size": c["vocab"], "hidden_size": d, "scale": 1.0}),
                             layers, default_schedule(3), norm("final."),
                             PartSpec("lm_head", "head.", {"vocab_size": c["vocab"], "hidden_size": d, "logit_scale": 1.0}))

    register_architecture(["toy-latent-arch"], LatentConfig)


def _toy_latent_plain(model, cfg, tokens):
    T, nh, dh, L = len(tokens), cfg["heads"], cfg["head_dim"], cfg["latent"]
    half = dh // 2
    cpu = lambda t: t.detach().cpu().double()
    sin, cos = P.plain_rope_tables(dh, 500.0, T)

    def rope(x):
        s, c = sin[:T, None, :], cos[:T, None, :]
        return torch.cat([x[..., :half] * c - x[..., half:] * s, x[..., :half] * s + x[..., half:] * c], -1)

    causal = torch.tril(torch.ones(T, T, dtype=torch.bool))
    x = P.plain_embedding(cpu(model.embedding.table), tokens, 1.0)
    for blk in model.layers:
        h = P.plain_rmsnorm(x, cpu(blk.mixer_norm.weight), 1e-5)
        m = blk.mixer
        if hasattr(m, "w_down"):
            c = P.plain_linear(h, cpu(m.w_down))
            p = torch.softmax((c @ c.t() / L ** 0.5).masked_fill(~causal, float("-inf")), -1)
            mean = torch.cumsum(c, 0) / torch.arange(1, T + 1)[:, None]
            y = P.plain_linear(p @ c + mean, cpu(m.w_up))
        else:
            qkv = P.plain_linear(h, cpu(m.w_qkv))
            q = rope(qkv[:, :nh * dh].reshape(T, nh, dh))
            k = rope(qkv[:, nh * dh:(nh + 1) * dh].reshape(T, 1, dh))
            v = qkv[:, (nh + 1) * dh:].reshape(T, 1, dh)
            y = P.plain_linear(P.plain_attention(q, k, v, dh ** -0.5, 0, None).reshape(T, nh * dh), cpu(m.w_o))
        x = x + 0.7 * y
        h = P.plain_rmsnorm(x, cpu(blk.feed_forward_norm.weight), 1e-5)
        gu = P.plain_linear(h, cpu(blk.feed_forward.w_gate_up))
        di = gu.shape[1] // 2
        x = x + 0.7 * P.plain_linear(P.plain_swiglu(gu[:, :di], gu[:, di:]), cpu(blk.feed_forward.w_down))
    return P.plain_linear(P.plain_rmsnorm(x, cpu(model.final_norm.weight), 1e-5), cpu(model.head.weight))


def test_toy_architecture_with_a_one_plane_latent_cache_and_a_state_in_one_mixer():
    """A mixer that asks for paged memory of one plane (a latent vector per token) AND a fixed-size state,
    beside the package's attention with its keys and values: two cache groups of different plane counts,
    pages given back and used again, a forked request, no change to the framework's files."""
    from infinicore_infer_amd.config import config_from_dict
    from infinicore_infer_amd.engine import Engine, StepEntry
    from infinicore_infer_amd.parts import Runtime, build_model
    from infinicore_infer_amd.weights import init_random_weights
    _register_toy_latent()
    cfg = {"model_type": "toy-latent-arch", "vocab": 83, "hidden": 56, "heads": 3, "head_dim": 32, "latent": 24, "inner": 72,
           "max_pos": 192}
    model = build_model(config_from_dict(cfg).model_spec(), Runtime(torch.float32, DEV))
    init_random_weights(model, seed=23, std=0.2, norm_std=0.1, tie=False)
    needs = model.cache_needs()
    assert [(n.kind, n.planes if n.paged else 0) for n in needs] == [("kv+state", 1), ("kv", 2), ("kv+state", 1)]
    requests = {"z%d" % i: H.random_tokens(83, n, 80 + i) for i, n in enumerate([66, 21, 110, 5])}
    ref = {rid: _toy_latent_plain(model, cfg, toks) for rid, toks in requests.items()}
    for maker in (H.trace_whole, H.trace_chunks, H.trace_mixed):
        steps, max_tokens = maker(requests)
        eng = Engine(model, max_tokens=max_tokens, page_size=16, max_requests=4)
        assert sorted((g.planes, g.n_kv_heads, g.head_dim, len(g.slots)) for g in eng.groups) == [(1, 1, 24, 2), (2, 1, 32, 1)]
        assert eng.native is None and not eng.use_graphs and eng.has_state
        assert [tuple(p.shape[:2]) for p in eng.storage.group_planes] in ([(2, 1), (1, 2)], [(1, 2), (2, 1)])
        got = H.run_trace(eng, steps)
        H.compare(got, ref, 1e-4, "toy latent %s" % maker.__name__)
        eng.cache.check_invariants()
        assert all(eng.cache.free_pages(g) == eng.num_pages for g in range(2))
    # a fork copies the pages of both groups and the state: the copy goes on as the original would
    toks = requests["z2"]
    eng = Engine(model, max_tokens=512, page_size=16, max_requests=4)
    eng.step([StepEntry("src", toks[:70], [])])
    eng.fork("src", "dst")
    eng.step([StepEntry("src", H.random_tokens(83, 9, 1), [])])          # the original moves on with other tokens
    out = eng.step([StepEntry("dst", toks[70:], list(range(len(toks) - 70)))])
    err = float((out.cpu().double() - ref["z2"][70:]).abs().max() / ref["z2"].abs().max())
    assert err < 1e-4, err


# ---------------------------------------------------------------------------
# a fourth toy architecture: layers that leave parts out.  A layer of a mixer alone (no feed-forward, no second
# norm) under the package's pre-norm block; and a block arrangement defined here that shares ONE norm between its
# mixer and its feed-forward (both read norm(x), both are added to the stream)
# ---------------------------------------------------------------------------
def _register_toy_sparse_layers():
    from infinicore_infer_amd.config import LayerSpec, ModelSpec, PartSpec, default_schedule, register_architecture
    from infinicore_infer_amd.kernels import ops
    from infinicore_infer_amd.parts import Block, register_part

    @register_part("block", "toy_parallel_one_norm")
    class ParallelBlock(Block):
        """x += a * (mixer(norm(x)) + ffn(norm(x))): one norm, no feed_forward_norm."""

        def __init__(self, name, runtime, mixer=None, mixer_norm=None, feed_forward=None, feed_forward_norm=None, a=1.0):
            super().__init__(name, runtime, mixer, mixer_norm, feed_forward, feed_forward_norm)
            assert feed_forward_norm is None and None not in (mixer, mixer_norm, feed_forward)
            self.a = float(a)

        def forward(self, x, pending, ctx, cache):
            if pending is not None:
                ops.residual_add(x, pending[0], pending[1])
            h = ctx.ws.buffer("toy_par_normed", tuple(x.shape), self.runtime.dtype)
            self.mixer_norm.forward(x, h)
            y = self.mixer.forward(h, ctx, cache)
            ops.residual_add(x, y, self.a)
            return (self.feed_forward.forward(h, ctx), self.a)          # the second add is left owed, as the package's block does

    class SparseConfig:
        def __init__(self, cfg):
            self.cfg = cfg

        @classmethod
        def from_dict(cls, cfg, **kw):
            return cls(cfg)

        def model_spec(self):
            c = self.cfg
            d, nh, nkvh, dh = c["hidden"], c["heads"], c["kv_heads"], c["head_dim"]
            rot = PartSpec("rotary", "", {"head_dim": dh, "theta": 500.0, "max_positions": c["max_pos"]})
            norm = lambda p: PartSpec("rmsnorm", p, {"size": d, "eps": 1e-5})
            ffn = lambda p: PartSpec("swiglu", p, {"hidden_size": d, "intermediate_size": c["inter"]})
            attn = lambda p: PartSpec("attention", p, {"hidden_size": d, "num_heads": nh, "num_kv_heads": nkvh, "head_dim": dh,
                                                       "softmax_scale": dh ** -0.5, "position_encoding": rot})
            pre = lambda p: PartSpec("prenorm_residual", p, {"residual_scale": 0.7})
            layers = [
                LayerSpec(pre("l0."), attn("l0.att."), norm("l0.n1.")),                                   # a mixer alone
                LayerSpec(pre("l1."), attn("l1.att."), norm("l1.n1.")),                                   # and another
                LayerSpec(pre("l2."), attn("l2.att."), norm("l2.n1."), ffn("l2.ffn."), norm("l2.n2.")),   # the usual layer
                LayerSpec(PartSpec("toy_parallel_one_norm", "l3.", {"a": 0.5}), attn("l3.att."), norm("l3.n."), ffn("l3.ffn.")),
                LayerSpec(pre("l4."), attn("l4.att."), norm("l4.n1.")),                                   # a mixer alone before the head
            ]
            return ModelSpec("toy-sparse", c["vocab"], d, c["max_pos"],
                             PartSpec("embedding", "emb.", {"vocab_size": c["vocab"], "hidden_size": d, "scale": 3.0}),
                             layers, default_schedule(len(layers)), norm("final."),
                             PartSpec("lm_head", "head.", {"vocab_size": c["vocab"], "hidden_size": d, "logit_scale": 1.0}))

    register_architecture(["toy-sparse-arch"], SparseConfig)


def _toy_sparse_plain(model, cfg, tokens, rnd=None):
    rnd = rnd or (lambda t: t)
    T, d, nh, nkvh, dh = len(tokens), cfg["hidden"], cfg["heads"], cfg["kv_heads"], cfg["head_dim"]
    half = dh // 2
    cpu = lambda t: t.detach().cpu().double()
    sin, cos = P.plain_rope_tables(dh, 500.0, T)

    def rope(x):
        s, c = sin[:T, None, :], cos[:T, None, :]
        return torch.cat([x[..., :half] * c - x[..., half:] * s, x[..., :half] * s + x[..., half:] * c], -1)

    def attention(blk, h):
        qkv = rnd(P.plain_linear(h, cpu(blk.mixer.w_qkv)))
        q = rnd(rope(qkv[:, :nh * dh].reshape(T, nh, dh)))
        k = rnd(rope(qkv[:, nh * dh:(nh + nkvh) * dh].reshape(T, nkvh, dh)))
        v = qkv[:, (nh + nkvh) * dh:].reshape(T, nkvh, dh)
        a = rnd(P.plain_attention(q, k, v, dh ** -0.5, 0, None)).reshape(T, nh * dh)
        return rnd(P.plain_linear(a, cpu(blk.mixer.w_o)))

    def ffn(blk, h):
        gu = rnd(P.plain_linear(h, cpu(blk.feed_forward.w_gate_up)))
        di = gu.shape[1] // 2
        return rnd(P.plain_linear(rnd(P.plain_swiglu(gu[:, :di], gu[:, di:])), cpu(blk.feed_forward.w_down)))

    x = P.plain_embedding(cpu(model.embedding.table), tokens, 3.0)
    for blk in model.layers:
        h = rnd(P.plain_rmsnorm(x, cpu(blk.mixer_norm.weight), 1e-5))
        if type(blk).__name__ == "ParallelBlock":
            x = x + 0.5 * attention(blk, h) + 0.5 * ffn(blk, h)
            continue
        x = x + 0.7 * attention(blk, h)
        if blk.feed_forward is not None:
            x = x + 0.7 * ffn(blk, rnd(P.plain_rmsnorm(x, cpu(blk.feed_forward_norm.weight), 1e-5)))
    return P.plain_linear(rnd(P.plain_rmsnorm(x, cpu(model.final_norm.weight), 1e-5)), cpu(model.head.weight))


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-4), (torch.bfloat16, H.BF16_TOL)])
def test_toy_architecture_whose_layers_leave_parts_out(dtype, tol):
    """Layers of a mixer alone under the package's own block (in bfloat16 with few rows their adds and norms still go
    into the products on either side: the mixer's last projection hands half-normed rows to the next layer's mixer,
    or to the head), and a block defined here with one norm for both its parts."""
    from infinicore_infer_amd.config import config_from_dict
    from infinicore_infer_amd.engine import Engine
    from infinicore_infer_amd.parts import Runtime, build_model
    from infinicore_infer_amd.weights import init_random_weights
    _register_toy_sparse_layers()
    cfg = {"model_type": "toy-sparse-arch", "vocab": 83, "hidden": 64, "heads": 4, "kv_heads": 2, "head_dim": 32,
           "inter": 96, "max_pos": 192}
    model = build_model(config_from_dict(cfg).model_spec(), Runtime(dtype, DEV))
    init_random_weights(model, seed=17, std=0.12, norm_std=0.1, tie=False)
    assert [l.feed_forward is None for l in model.layers] == [True, True, False, False, True]
    assert model.layers[3].feed_forward_norm is None and len(model.cache_needs()) == 5
    requests = {"s%d" % i: H.random_tokens(83, n, 80 + i) for i, n in enumerate([60, 21, 130, 7])}
    rnd = P.round_bf16 if dtype == torch.bfloat16 else None
    ref = {rid: _toy_sparse_plain(model, cfg, toks, rnd) for rid, toks in requests.items()}
    for maker in (H.trace_whole, H.trace_last_one_by_one, H.trace_mixed):
        steps, max_tokens = maker(requests)
        eng = Engine(model, max_tokens=max_tokens, page_size=16, max_requests=4)
        assert eng.native is None                      # a layer without a feed-forward has no native description
        H.compare(H.run_trace(eng, steps), ref, tol, "toy sparse layers %s" % maker.__name__, steps=steps)
        eng.cache.check_invariants()
