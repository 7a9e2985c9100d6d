"""The plain implementation is pinned by what fixes it beside the reference's text:
library routines for special cases and invariants, each chosen so that a plausible
mistake fails it.  The reference holds no test vectors (it has no tests directory and
no stored outputs), so agreement with real checkpoints is parity unpinned. (CPU)"""
import math

import pytest
import torch
import torch.nn.functional as F

import helpers as H
import plain_model as P

torch.manual_seed(0)


def test_rmsnorm_is_the_library_routine_and_eps_sits_inside_the_root():
    x = torch.randn(5, 96, dtype=torch.float64)
    w = torch.randn(96, dtype=torch.float64)
    assert torch.allclose(P.plain_rmsnorm(x, w, 1e-6), F.rms_norm(x, (96,), w, 1e-6), atol=1e-12)
    tiny = torch.full((1, 8), 1e-4, dtype=torch.float64)
    y5 = P.plain_rmsnorm(tiny, torch.ones(8), 1e-5)
    y6 = P.plain_rmsnorm(tiny, torch.ones(8), 1e-6)
    assert float(y5[0, 0]) == pytest.approx(1e-4 / math.sqrt(1e-8 + 1e-5))
    assert float(y6[0, 0]) == pytest.approx(1e-4 / math.sqrt(1e-8 + 1e-6))
    ones = P.plain_rmsnorm(x, torch.ones(96), 1e-5)
    m = (x * x).mean(-1)
    assert torch.allclose((ones * ones).mean(-1), m / (m + 1e-5))


def test_rope_special_cases():
    sin, cos = P.plain_rope_tables(2, 10000.0, 8)
    x = torch.randn(8, 1, 2, dtype=torch.float64)
    y = P.plain_rope_adjacent(x, list(range(8)), sin, cos)
    assert torch.allclose(y[0], x[0])                                   # position 0 is the identity
    for p in range(8):                                                  # head size 2: a plane rotation by p radians
        rot = torch.tensor([[math.cos(p), -math.sin(p)], [math.sin(p), math.cos(p)]], dtype=torch.float64)
        assert torch.allclose(y[p, 0], rot @ x[p, 0])
    s4, c4 = P.plain_rope_tables(16, 1e4, 50)
    s6, c6 = P.plain_rope_tables(16, 1e6, 50)
    assert torch.allclose(s4[:, 0], s6[:, 0]) and not torch.allclose(s4[:, 3], s6[:, 3])
    assert float(s4[7, 2]) == pytest.approx(math.sin(7 / 1e4 ** (2 / 8)))   # jiuge_weight.hpp:141-142
    sf, cf = P.plain_rope_tables(16, 1e4, 50, factors=[1.0] * 8, magnitude=1.0)
    assert torch.equal(sf, s4) and torch.equal(cf, c4)                  # neutral long-context scaling = plain


def test_rope_keeps_norms_and_only_distances_count():
    dh = 32
    sin, cos = P.plain_rope_tables(dh, 1e4, 300)
    q = torch.randn(1, 1, dh, dtype=torch.float64)
    k = torch.randn(1, 1, dh, dtype=torch.float64)

    def score(m, n):
        return float((P.plain_rope_adjacent(q, [m], sin, cos) * P.plain_rope_adjacent(k, [n], sin, cos)).sum())

    assert score(10, 3) == pytest.approx(score(110, 103), abs=1e-9)     # a wrong sign breaks this
    assert score(10, 3) != pytest.approx(score(3, 10), abs=1e-6)
    r = P.plain_rope_adjacent(q, [77], sin, cos)
    assert torch.allclose((r[..., 0::2] ** 2 + r[..., 1::2] ** 2), (q[..., 0::2] ** 2 + q[..., 1::2] ** 2))


def test_adjacent_pairs_on_permuted_rows_equal_half_split_pairs():
    """scripts/jiuge.py:217-227: the host permutation turns pairs (j, j+dh/2) into (2j, 2j+1)."""
    nh, dh, d = 3, 16, 24
    w = torch.randn(nh * dh, d, dtype=torch.float64)
    h = torch.randn(5, d, dtype=torch.float64)
    sin, cos = P.plain_rope_tables(dh, 1e4, 64)
    pos = [0, 9, 17, 33, 63]
    wp = P.permute_rows_to_adjacent_pairs(w, nh, dh)
    a = P.plain_rope_adjacent(P.plain_linear(h, wp).reshape(5, nh, dh), pos, sin, cos)
    x = P.plain_linear(h, w).reshape(5, nh, dh)
    half = dh // 2
    s, c = sin[pos][:, None, :], cos[pos][:, None, :]
    b = torch.cat([x[..., :half] * c - x[..., half:] * s, x[..., :half] * s + x[..., half:] * c], -1)
    # same numbers, pair j of b sits at (j, j+half), of a at (2j, 2j+1): all dot products agree
    assert torch.allclose(a[..., 0::2], b[..., :half]) and torch.allclose(a[..., 1::2], b[..., half:])


def test_attention_special_cases_and_library_routine():
    s, nh, nkvh, dh, past = 6, 4, 2, 16, 5
    t = past + s
    q = torch.randn(s, nh, dh, dtype=torch.float64)
    k = torch.randn(t, nkvh, dh, dtype=torch.float64)
    v = torch.randn(t, nkvh, dh, dtype=torch.float64)
    scale = 1 / math.sqrt(dh)
    out = P.plain_attention(q, k, v, scale, past)
    # library attention with an explicit bottom-right mask, kv heads repeated per group (GQA = MHA on repeats)
    mask = torch.arange(t)[None, :] <= past + torch.arange(s)[:, None]
    kk = k.repeat_interleave(nh // nkvh, dim=1).transpose(0, 1)
    vv = v.repeat_interleave(nh // nkvh, dim=1).transpose(0, 1)
    lib = F.scaled_dot_product_attention(q.transpose(0, 1), kk, vv, attn_mask=mask, scale=scale).transpose(0, 1)
    assert torch.allclose(out, lib, atol=1e-12)
    # a top-left aligned mask (the plausible mistake) differs
    bad = torch.arange(t)[None, :] <= torch.arange(s)[:, None]
    lib_bad = F.scaled_dot_product_attention(q.transpose(0, 1), kk, vv, attn_mask=bad, scale=scale).transpose(0, 1)
    assert not torch.allclose(out, lib_bad, atol=1e-3)
    one = P.plain_attention(q[:1], k[:1], v[:1], scale, 0)
    assert torch.allclose(one[0, 0], v[0, 0]) and torch.allclose(one[0, 3], v[0, 1])      # head 3 -> kv head 1
    mean = P.plain_attention(torch.zeros(1, nh, dh, dtype=torch.float64), k, v, scale, t - 1)
    assert torch.allclose(mean[0, 0], v[:, 0].mean(0))
    w = P.plain_attention(q, k, v, scale, past, window=3)
    assert torch.allclose(w[-1, 0], P.plain_attention(q[-1:], k[-3:], v[-3:], scale, 2)[0, 0])
    assert not torch.allclose(P.plain_attention(q, k, v, 1.0, past), out)                 # the scale matters


def test_swiglu_argument_order():
    g = torch.randn(4, 10, dtype=torch.float64)
    u = torch.randn(4, 10, dtype=torch.float64)
    assert torch.allclose(P.plain_swiglu(g, u), F.silu(g) * u)
    assert not torch.allclose(P.plain_swiglu(g, u), F.silu(u) * g)
    assert torch.all(P.plain_swiglu(torch.zeros_like(g), u) == 0)


def _weights(name, seed=0):
    from infinicore_infer_amd.weights import random_state_dict
    cfg, init = H.CONFIGS[name]
    return cfg, random_state_dict(cfg, seed, dtype=torch.float32, **init)


def test_neutral_constants_are_the_plain_llama_graph():
    """scale_emb = 1, scale_depth = sqrt(L), dim_model_base = hidden gives the graph without the
    constants (the reference's own fallback, scripts/jiuge.py:97-106)."""
    cfg, sd = _weights("A")
    toks = H.random_tokens(256, 12, 1)
    neutral = dict(cfg, scale_emb=1.0, scale_depth=math.sqrt(2), dim_model_base=64)
    bare = {k: v for k, v in cfg.items() if k not in ("scale_emb", "scale_depth", "dim_model_base")}
    assert torch.allclose(P.plain_forward(neutral, sd, toks), P.plain_forward(bare, sd, toks), atol=1e-12)
    assert not torch.allclose(P.plain_forward(cfg, sd, toks), P.plain_forward(bare, sd, toks), atol=1e-3)


def test_logit_scale_direction_and_host_folding():
    """Tiny A has width ratio 4: the reference multiplies (jiuge.py:108,199).  Folding the constants
    into the weights on the host, as jiuge.py:195,199,297,348 does, gives the same logits."""
    cfg, sd = _weights("A")
    toks = H.random_tokens(256, 9, 2)
    ref = P.plain_forward(cfg, sd, toks)
    mup = P.plain_forward(cfg, sd, toks, logit_scale_rule="mup")
    assert torch.allclose(ref, mup * 16.0, rtol=1e-9)
    s_in, s_out, s_res = P.plain_scales(cfg)
    assert (s_in, s_out) == (12.0, 4.0) and s_res == pytest.approx(1.4 / math.sqrt(2))
    folded = {k: v.double().clone() for k, v in sd.items()}
    folded["lm_head.weight"] = folded["model.embed_tokens.weight"].clone()
    folded["model.embed_tokens.weight"] *= s_in
    folded["model.norm.weight"] *= s_out
    for l in range(2):
        folded["model.layers.%d.self_attn.o_proj.weight" % l] *= s_res
        folded["model.layers.%d.mlp.down_proj.weight" % l] *= s_res
    bare = {k: v for k, v in cfg.items() if k not in ("scale_emb", "scale_depth", "dim_model_base")}
    assert torch.allclose(P.plain_forward(bare, folded, toks), ref, atol=1e-9)


def test_causality_shift_invariance_and_tying():
    cfg, sd = _weights("B")
    toks = H.random_tokens(509, 20, 3)
    full = P.plain_forward(cfg, sd, toks)
    changed = toks[:10] + [(t + 1) % 509 for t in toks[10:]]
    assert torch.allclose(P.plain_forward(cfg, sd, changed)[:10], full[:10], atol=1e-12)
    assert torch.allclose(P.plain_forward(cfg, sd, toks[:7]), full[:7], atol=1e-10)
    # only distances between positions count (rotary): shifting every position changes nothing
    assert torch.allclose(P.plain_forward(cfg, sd, toks, start_pos=37), full, atol=1e-9)
    # an untied head that is a copy of the embedding = the tied model
    cfg_a, sd_a = _weights("A")
    toks_a = [t % 256 for t in toks[:8]]
    tied = P.plain_forward(cfg_a, sd_a, toks_a)
    untied = dict(sd_a, **{"lm_head.weight": sd_a["model.embed_tokens.weight"].clone()})
    assert torch.equal(P.plain_forward(cfg_a, untied, toks_a), tied)


def test_fused_projections_equal_separate_ones():
    h = torch.randn(4, 24, dtype=torch.float64)
    a, b, c = (torch.randn(8, 24, dtype=torch.float64) for _ in range(3))
    fused = P.plain_linear(h, torch.cat([a, b, c]))
    assert torch.allclose(fused, torch.cat([P.plain_linear(h, a), P.plain_linear(h, b), P.plain_linear(h, c)], 1))
    assert torch.allclose(P.plain_linear(h, a), F.linear(h, a))


def test_plain_sampling_rules():
    z = torch.tensor([0.1, 2.0, -1.0, 2.0, 0.5], dtype=torch.float64)
    assert P.plain_sample(z, 0.0, 0, 1.0, 0.7) == 1 and P.plain_sample(z, 1.0, 1, 1.0, 0.7) == 1
    p = torch.softmax(z, 0)
    cdf = torch.cumsum(p, 0)
    for u in (0.0, 0.05, 0.3, 0.62, 0.9, 0.999):
        want = int(torch.nonzero(cdf >= u * float(cdf[-1]))[0])
        assert P.plain_sample(z, 1.0, 0, 1.0, u) == want == P.plain_sample(z, 1.0, 5, 1.0, u)
    assert {P.plain_sample(z, 1.0, 2, 1.0, u) for u in (0.01, 0.3, 0.6, 0.99)} == {1, 3}     # the two largest
    assert {P.plain_sample(z, 1.0, 0, 0.5, u) for u in (0.01, 0.3, 0.6, 0.99)} == {1, 3}     # equal values stay together
    assert P.plain_sample(z, 1.0, 0, 0.9, 0.999) == 4       # the two largest hold 0.826: 0.9 needs the third value
    assert P.plain_sample(z * 1000, 1.0, 0, 1.0, 0.0) == 1          # u = 0: the first token that has any mass
    cold = [P.plain_sample(z, 1e-4, 0, 1.0, u) for u in (0.1, 0.4)]
    assert set(cold) <= {1, 3}


def test_bf16_rounding_helper():
    x = torch.tensor([1.0, 1.00390625, 1.005859375, 3.14159], dtype=torch.float64)
    assert torch.equal(P.round_bf16(x), x.float().to(torch.bfloat16).double())
    assert float(P.round_bf16(torch.tensor([1.00390625], dtype=torch.float64))) == 1.0      # ties to even
