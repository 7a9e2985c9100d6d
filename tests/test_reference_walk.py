"""The two plain implementations pin each other: ``plain_model.plain_forward`` (whole sequences, constants at run
time, no cache) against ``reference_walk.ReferenceWalk`` (the reference's buffers step by step: folded constants,
permuted q/k rows, a cache slab per request, batches of (req_lens, req_pos)).  A mistake in either one's reading of
the composition (which stream a norm reads, where the residual is added, which kv head a query head uses, the
direction of the final scale) shows as a difference; each such mistake is put into a copy of the plain model below
and must be caught.  The long-context rotary scaling has no text in the reference: its rule is pinned by what it
must reduce to.  (CPU)"""
import math

import numpy as np
import pytest
import torch

import helpers as H
import plain_model as P
from reference_walk import ReferenceWalk


def _weights(name, seed=0):
    from infinicore_infer_amd.weights import random_state_dict
    cfg, init = H.CONFIGS[name]
    return cfg, random_state_dict(cfg, seed, dtype=torch.float32, **init)


def _walk_logits(cfg, sd, requests, first_portion):
    """Every request's prompt cut in two steps (so the second portion reads the cache), all requests in one batch,
    then three single-token steps: {(id, position): logits row} for the last token of every request in every step."""
    walk = ReferenceWalk(cfg, sd)
    caches = {rid: walk.create_kv_cache() for rid in requests}
    pos = {rid: 0 for rid in requests}
    out = {}

    def step(portions):
        ids = list(portions)
        tokens = [t for rid in ids for t in portions[rid]]
        logits = walk.infer_batch(tokens, [len(portions[rid]) for rid in ids], [pos[rid] for rid in ids],
                                  [caches[rid] for rid in ids])
        for i, rid in enumerate(ids):
            pos[rid] += len(portions[rid])
            out[(rid, pos[rid] - 1)] = logits[i]

    n_dec = 3
    step({rid: toks[:min(first_portion, len(toks) - n_dec - 1)] for rid, toks in requests.items()})
    step({rid: toks[pos[rid]:len(toks) - n_dec] for rid, toks in requests.items()})
    for j in range(n_dec):
        step({rid: [toks[len(toks) - n_dec + j]] for rid, toks in requests.items()})
    return out


def _worst(out, plain):
    return max(float(np.abs(row - plain[rid][p].numpy()).max()) / float(plain[rid].abs().max()) for (rid, p), row in out.items())


@pytest.mark.parametrize("name", ["A", "B"])
def test_the_walk_through_the_reference_equals_the_plain_model(name):
    cfg, sd = _weights(name)
    requests = {"r%d" % i: H.random_tokens(cfg["vocab_size"], n, 70 + i) for i, n in enumerate([9, 40, 17])}
    out = _walk_logits(cfg, sd, requests, first_portion=5)
    assert len(out) == 3 * 5
    plain = {rid: P.plain_forward(cfg, sd, toks) for rid, toks in requests.items()}
    assert _worst(out, plain) < 1e-9
    # forwardBatch: every row
    walk = ReferenceWalk(cfg, sd)
    toks = requests["r1"]
    every = walk.infer_batch(toks, [len(toks)], [0], [walk.create_kv_cache()], all_rows=True)
    assert float(np.abs(every - plain["r1"].numpy()).max()) / float(plain["r1"].abs().max()) < 1e-9


def test_mistakes_in_the_composition_are_caught(monkeypatch):
    """Each plausible misreading, put into the plain model, makes it differ from the walk."""
    cfg, sd = _weights("A")
    cfg = dict(cfg, scale_depth=3.0)             # (tiny A's own 1.4 / sqrt(2) is 0.99: a missing factor would not show)
    # with weights of 0.02 every score is near zero and attention is a plain mean, whatever the pairing, the head map or
    # the scale: the projections of q and k are scaled up so that the scores decide who is attended
    sd = {k: (v * 40.0 if ("q_proj" in k or "k_proj" in k) else v) for k, v in sd.items()}
    cfg_b, sd_b = _weights("B")
    requests = {"r0": H.random_tokens(256, 21, 5), "r1": H.random_tokens(256, 12, 6)}
    requests_b = {"r0": H.random_tokens(509, 21, 5), "r1": H.random_tokens(509, 12, 6)}
    out = _walk_logits(cfg, sd, requests, 6)
    out_b = _walk_logits(cfg_b, sd_b, requests_b, 6)

    def differs(out, cfg, sd, requests, **kw):
        return _worst(out, {rid: P.plain_forward(cfg, sd, toks, **kw) for rid, toks in requests.items()}) > 1e-3

    assert not differs(out, cfg, sd, requests) and not differs(out_b, cfg_b, sd_b, requests_b)
    # the two norms of a layer read each other's weights (tiny B has random norm weights)
    swapped = dict(sd_b)
    for l in range(cfg_b["num_hidden_layers"]):
        a, b = "model.layers.%d.input_layernorm.weight" % l, "model.layers.%d.post_attention_layernorm.weight" % l
        swapped[a], swapped[b] = sd_b[b], sd_b[a]
    assert differs(out_b, cfg_b, swapped, requests_b)
    # the final scale divides instead of multiplying (tiny A: width ratio 4)
    assert differs(out, cfg, sd, requests, logit_scale_rule="mup")
    # query head h reads kv head h % nkvh instead of h // group (tiny A: 4 query heads on 2 kv heads)
    true_attention = P.plain_attention

    def interleaved(q, k, v, scale, past=0, window=None):
        nh, nkvh = q.shape[1], k.shape[1]
        kk = torch.stack([k[:, h % nkvh] for h in range(nh)], 1)        # one kv head per query head, chosen the wrong way
        vv = torch.stack([v[:, h % nkvh] for h in range(nh)], 1)
        return true_attention(q, kk, vv, scale, past, window)
    monkeypatch.setattr(P, "plain_attention", interleaved)
    assert differs(out, cfg, sd, requests)
    monkeypatch.undo()
    # gate and up swapped in the activation
    true_swiglu = P.plain_swiglu
    monkeypatch.setattr(P, "plain_swiglu", lambda gate, up: true_swiglu(up, gate))
    assert differs(out, cfg, sd, requests)
    monkeypatch.undo()
    # the residual branches not scaled by scale_depth / sqrt(L)
    true_scales = P.plain_scales
    monkeypatch.setattr(P, "plain_scales", lambda c, rule="reference": true_scales(c, rule)[:2] + (1.0,))
    assert differs(out, cfg, sd, requests)
    monkeypatch.undo()
    # the embedding not scaled by scale_emb
    monkeypatch.setattr(P, "plain_scales", lambda c, rule="reference": (1.0,) + true_scales(c, rule)[1:])
    assert differs(out, cfg, sd, requests)
    monkeypatch.undo()
    # rotary pairs taken as adjacent rows of the checkpoint's own order (no host permutation)
    monkeypatch.setattr(P, "permute_rows_to_adjacent_pairs", lambda w, n, dh: w)
    assert differs(out, cfg, sd, requests)
    monkeypatch.undo()
    # the softmax scale 1 / dh instead of 1 / sqrt(dh)
    monkeypatch.setattr(P, "plain_attention", lambda q, k, v, scale, past=0, window=None: true_attention(q, k, v, scale * scale, past, window))
    assert differs(out, cfg, sd, requests)
    monkeypatch.undo()
    # the post-attention norm reads the stream from before the attention's residual add
    true_norm = P.plain_rmsnorm
    seen = []

    def stale_norm(x, w, eps):
        seen.append(x)
        if len(seen) % 2 == 0 and len(seen) <= 2 * cfg["num_hidden_layers"]:      # every second norm of a layer: the pre-FFN one
            return true_norm(seen[-2], w, eps)
        return true_norm(x, w, eps)
    monkeypatch.setattr(P, "plain_rmsnorm", stale_norm)
    bad = P.plain_forward(cfg, sd, requests["r0"])
    monkeypatch.undo()
    good = P.plain_forward(cfg, sd, requests["r0"])
    assert float((bad - good).abs().max()) / float(good.abs().max()) > 1e-3 and _worst({k: v for k, v in out.items() if k[0] == "r0"}, {"r0": bad}) > 1e-3
    assert not differs(out, cfg, sd, requests)


def test_the_walk_checks_the_plain_models_mask_alignment():
    """A mask aligned to the top left (row i of a portion sees keys <= i instead of <= past + i) is a mistake that
    whole sequences cannot show (past = 0).  The walk's second portions and single tokens read a cache: its causal
    softmax [nh, seq_len, total_len] must let the last row see every key (jiuge.cpp:225-226)."""
    s = np.random.RandomState(0).randn(2, 3, 7)
    p = ReferenceWalk._causal_softmax(s)
    assert np.allclose(p.sum(-1), 1.0)
    assert np.all(p[:, 0, 5:] == 0) and np.all(p[:, 0, :5] > 0) and np.all(p[:, 2] > 0)
    lib = torch.softmax(torch.from_numpy(s).masked_fill(~(torch.arange(7)[None, :] <= 4 + torch.arange(3)[:, None]), float("-inf")), -1)
    assert np.allclose(p, lib.numpy())


# ---- long-context rotary scaling: no text in the reference; pinned by what it must reduce to --------------------------
def test_longrope_rule():
    """angle = p / (factor_j * theta^(j / half)); the long factors and the magnitude sqrt(1 + ln(ratio) / ln(original))
    apply when the configured context exceeds the original one, else the short factors and magnitude 1.  The rule is
    this engine's own (parity unpinned: the reference reads no rope_scaling); what fixes it here: a constant factor c
    is the plain table read at position p / c; the choice between the arrays and the magnitude's value by hand."""
    dh, theta = 16, 10000.0
    s1, c1 = P.plain_rope_tables(dh, theta, 40)
    s3, c3 = P.plain_rope_tables(dh, theta, 120, factors=[3.0] * 8)
    assert torch.allclose(s3[0::3], s1, atol=1e-12) and torch.allclose(c3[0::3], c1, atol=1e-12)
    # a factor on one pair only slows that pair and leaves the others alone
    f = [1.0] * 8
    f[2] = 2.0
    s2, c2 = P.plain_rope_tables(dh, theta, 80, factors=f)
    plain_s, _ = P.plain_rope_tables(dh, theta, 80)
    assert torch.allclose(s2[0::2, 2], plain_s[:40, 2], atol=1e-12) and torch.equal(s2[:, 3], plain_s[:, 3])
    sm, cm = P.plain_rope_tables(dh, theta, 40, magnitude=1.25)
    assert torch.allclose(sm, 1.25 * s1) and torch.allclose(cm, 1.25 * c1)
    scaling = dict(type="longrope", original_max_position_embeddings=4096, short_factor=[1.5] * 8, long_factor=[2.5] * 8)
    longer = dict(max_position_embeddings=32768, rope_scaling=scaling)
    same = dict(max_position_embeddings=4096, rope_scaling=scaling)
    shorter = dict(max_position_embeddings=2048, rope_scaling=scaling)
    assert P.plain_longrope(longer) == ([2.5] * 8, pytest.approx(math.sqrt(1.0 + math.log(8.0) / math.log(4096.0))))
    assert P.plain_longrope(longer)[1] == pytest.approx(1.1180339887)          # sqrt(1 + 3/12): ln 8 / ln 4096 = 1/4
    assert P.plain_longrope(same) == ([1.5] * 8, 1.0) and P.plain_longrope(shorter) == ([1.5] * 8, 1.0)
    assert P.plain_longrope(dict(max_position_embeddings=128)) == (None, 1.0)


@pytest.mark.parametrize("which", ["C", "wide", "8b"])
def test_the_engines_rotary_tables_equal_the_plain_ones(which):
    """The package's table builder against the plain one, for tiny C, the wide test shape and the benchmark's 8B
    configuration (context = original: short factors, magnitude 1), also under a serving cap on the context."""
    from infinicore_infer_amd.parts.rotary import rotary_tables
    if which == "C":
        cfg, dh = H.TINY_C, 64
    elif which == "wide":
        cfg = dict(max_position_embeddings=512, rope_theta=10000.0,
                   rope_scaling=dict(type="longrope", original_max_position_embeddings=128,
                                     short_factor=[1.0 + 3.0 * i / 63 for i in range(64)],
                                     long_factor=[1.0 + 2.0 * ((7 * i) % 64) / 63 for i in range(64)]))
        dh = 128
    else:
        cfg = dict(max_position_embeddings=32768, rope_theta=10000.0,
                   rope_scaling=dict(type="longrope", original_max_position_embeddings=32768,
                                     short_factor=[1.0 + 0.04 * i for i in range(64)], long_factor=[2.0 + 0.03 * i for i in range(64)]))
        dh = 128
    factors, magnitude = P.plain_longrope(cfg)
    n = min(cfg["max_position_embeddings"], 1024)
    sin, cos = P.plain_rope_tables(dh, cfg["rope_theta"], n, factors, magnitude)
    c, s = rotary_tables(dh, cfg["rope_theta"], n, cfg["rope_scaling"], model_max_positions=cfg["max_position_embeddings"])
    assert torch.allclose(c.double(), cos, atol=1e-6) and torch.allclose(s.double(), sin, atol=1e-6)
    if which == "wide":
        assert factors == cfg["rope_scaling"]["long_factor"] and magnitude > 1.0
    if which == "8b":
        assert factors == cfg["rope_scaling"]["short_factor"] and magnitude == 1.0
