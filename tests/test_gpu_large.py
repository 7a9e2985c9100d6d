"""The shapes and schedules that the benchmark measures, against the plain implementation: the whole
MiniCPM-2B-shaped model (40 layers, vocabulary 122,753) with a 2,048-token prompt, decoding one by one, and 64 live
requests over 2,048..2,100 keys; two layers of the 8B shape with a 16,384-token prompt whole and in portions and
decoding over 16,400 keys; two layers of the 1B shape with 64 live requests, some 50 single tokens beside two portions
of 512 in a step, and pages that are used again.  The engine's loop these must equal is the reference's
src/models/jiuge/jiuge.cpp:205-233 (per request: past_len + seq_len keys).

The plain implementation computes the same float64 mathematics as everywhere, with its tensors on the GPU (the
same torch operations, only faster); only the wanted positions go through the head.  Weights are drawn from the seed
by the package's generator twice: straight into the engine's model, and by checkpoint name for the plain model (a
value is a function of seed, tensor name and element index alone)."""
import random

import pytest
import torch

import helpers as H

pytestmark = pytest.mark.gpu
DEV = "cuda:0"

SHAPE_2B = dict(model_type="minicpm", vocab_size=122753, hidden_size=2304, num_hidden_layers=40, num_attention_heads=36,
                num_key_value_heads=36, intermediate_size=5760, max_position_embeddings=4096, rms_norm_eps=1e-5,
                rope_theta=10000.0, scale_emb=12, dim_model_base=256, scale_depth=1.4, tie_word_embeddings=True, eos_token_id=2)
SHAPE_1B = dict(SHAPE_2B, vocab_size=73440, hidden_size=1536, num_hidden_layers=2, num_attention_heads=24,
                num_key_value_heads=8, intermediate_size=3840)
_rng = random.Random(5)
SHAPE_8B = dict(SHAPE_2B, vocab_size=73448, hidden_size=4096, num_hidden_layers=2, num_attention_heads=32, num_key_value_heads=2,
                intermediate_size=16384, rms_norm_eps=1e-6, tie_word_embeddings=False, max_position_embeddings=32768,
                rope_scaling=dict(type="longrope", original_max_position_embeddings=4096,
                                  short_factor=[1.0 + 3.0 * _rng.random() for _ in range(64)],
                                  long_factor=[1.0 + 3.0 * _rng.random() for _ in range(64)]))


def _engine_and_weights(cfg, seed, std, max_tokens, max_requests, page_size=64, dtype=torch.bfloat16, **kw):
    from infinicore_infer_amd.config import config_from_dict
    from infinicore_infer_amd.engine import Engine
    from infinicore_infer_amd.parts import Runtime, build_model
    from infinicore_infer_amd.weights import init_random_weights, random_state_dict
    tie = bool(cfg.get("tie_word_embeddings", True))
    model = build_model(config_from_dict(cfg).model_spec(), Runtime(dtype=dtype, device=DEV))
    init_random_weights(model, seed=seed, std=std, norm_std=0.1, tie=tie)
    sd = random_state_dict(cfg, seed, std=std, norm_std=0.1, dtype=dtype, device=DEV, tie=tie)
    return Engine(model, max_tokens=max_tokens, page_size=page_size, max_requests=max_requests, **kw), sd


def _plain_rows(cfg, sd, tokens, rows, bf16=True):
    """{position: plain logits row (float64, CPU)} of one request at the given positions."""
    from plain_model import plain_forward, round_bf16
    rows = sorted(set(rows))
    out = plain_forward(cfg, sd, tokens, rnd=round_bf16 if bf16 else None, rows=rows).cpu()
    return {p: out[i] for i, p in enumerate(rows)}


def _step(engine, entries):
    from infinicore_infer_amd.engine import StepEntry
    logits = engine.step([StepEntry(*e) for e in entries])
    n = sum(len(e[2]) for e in entries)
    assert (logits is None) == (n == 0) and (n == 0 or logits.shape[0] == n)
    return None if logits is None else logits.float().cpu()


def test_the_whole_2b_shaped_model(capsys):
    """40 layers, hidden 2,304, 36 heads of 64, vocabulary 122,753, bfloat16.  One request of 2,048 tokens in one step, then
    32 tokens one by one (the recorded step of batch 1); then 63 more requests with prompts of 2,048..2,100 tokens, and all
    64 decode three steps together (one key split, block tables of 33 pages, the sliced O and down products, the library's
    QKV and gate/up products, the recorded step of batch 64)."""
    torch.manual_seed(0)
    engine, sd = _engine_and_weights(SHAPE_2B, seed=11, std=0.02, max_tokens=64 * 2176, max_requests=64)
    V = SHAPE_2B["vocab_size"]
    got, ref = {}, {}
    solo = H.random_tokens(V, 2048 + 32, 100)
    rows = [0, 1, 63, 64, 1000, 2047]
    out = _step(engine, [("solo", solo[:2048], rows)])
    for i, p in enumerate(rows):
        got[("solo", p)] = out[i]
    for j in range(2048, 2080):
        got[("solo", j)] = _step(engine, [("solo", [solo[j]], [0])])[0]
    assert engine.graph_replays >= 29 and engine.native_steps >= 1
    for p, r in _plain_rows(SHAPE_2B, sd, solo, rows + list(range(2048, 2080))).items():
        ref[("solo", p)] = r
    worst = H.compare_places(got, ref, H.BF16_TOL, "2B shape, one request")
    with capsys.disabled():
        print("\n2B shape, 2,048 tokens whole then 32 one by one: worst error %.3g of the largest logit at %s" % worst)
    # 64 live requests: "solo" stays, 63 others join with prompts of 2,048..2,100 tokens
    lens = {"solo": 2080}
    toks = {"solo": solo + H.random_tokens(V, 3, 101)}
    for i in range(63):
        rid = "q%02d" % i
        lens[rid] = 2048 + (i * 37) % 53
        toks[rid] = H.random_tokens(V, lens[rid] + 3, 200 + i)
        _step(engine, [(rid, toks[rid][:lens[rid]], [])])
    got, ref = {}, {}
    ids = list(lens)
    replays = engine.graph_replays
    for j in range(3):
        out = _step(engine, [(rid, [toks[rid][lens[rid] + j]], [0]) for rid in ids])
        for i, rid in enumerate(ids):
            got[(rid, lens[rid] + j)] = out[i]
    assert engine.graph_replays - replays >= 1           # the shape came back: recorded, then replayed
    for rid in ids:
        for p, r in _plain_rows(SHAPE_2B, sd, toks[rid], [lens[rid] + j for j in range(3)]).items():
            ref[(rid, p)] = r
    worst = H.compare_places(got, ref, H.BF16_TOL, "2B shape, 64 live requests")
    with capsys.disabled():
        print("2B shape, 64 requests over 2,048..2,103 keys, three steps: worst error %.3g at %s" % worst)
    for rid in ids:
        engine.free(rid)
    engine.cache.check_invariants()


def test_two_layers_of_the_8b_shape_over_16384_tokens(capsys):
    """32 query heads on 2 kv heads of 128, hidden 4,096, inner size 16,384, longrope with the long factors (context 32,768
    over an original 4,096).  A prompt of 16,384 tokens in one step and the same prompt in portions of 2,048 (256 key tiles
    in the longest walk, walks cut in parts); then four requests decode three steps over 16,384..16,420 keys (the
    grouped-query kernel at head size 128 with the split count the cost model chooses there)."""
    engine, sd = _engine_and_weights(SHAPE_8B, seed=12, std=0.02, max_tokens=4 * 16512, max_requests=4)
    V = SHAPE_8B["vocab_size"]
    lens = {"whole": 16384, "cut": 16384, "c": 16390, "d": 16417}
    toks = {"whole": H.random_tokens(V, 16384 + 3, 300)}
    toks["cut"] = toks["whole"][:16384] + H.random_tokens(V, 3, 301)      # the same prompt, another continuation
    toks["c"] = H.random_tokens(V, lens["c"] + 3, 302)
    toks["d"] = H.random_tokens(V, lens["d"] + 3, 303)
    got, ref = {}, {}
    rows = [0, 2047, 2048, 8191, 12000, 16383]
    out = _step(engine, [("whole", toks["whole"][:16384], rows)])
    for i, p in enumerate(rows):
        got[("whole", p)] = out[i]
    for o in range(0, 16384, 2048):
        want = [p - o for p in rows if o <= p < o + 2048]
        out = _step(engine, [("cut", toks["cut"][o:o + 2048], want)])
        for i, w in enumerate(want):
            got[("cut", o + w)] = out[i]
    for rid, portion in (("c", 4096), ("d", 3000)):
        for o in range(0, lens[rid], portion):
            _step(engine, [(rid, toks[rid][o:min(o + portion, lens[rid])], [])])
    ids = list(lens)
    for j in range(3):
        out = _step(engine, [(rid, [toks[rid][lens[rid] + j]], [0]) for rid in ids])
        for i, rid in enumerate(ids):
            got[(rid, lens[rid] + j)] = out[i]
    for rid in ids:
        places = [lens[rid] + j for j in range(3)] + (rows if rid in ("whole", "cut") else [])
        for p, r in _plain_rows(SHAPE_8B, sd, toks[rid], places).items():
            ref[(rid, p)] = r
    worst = H.compare_places(got, ref, H.BF16_TOL, "8B shape, 16,384 tokens")
    with capsys.disabled():
        print("\n8B shape (2 layers), 16,384 tokens whole and in portions, 4 requests decoding: worst error %.3g at %s" % worst)
    for rid in ids:
        engine.free(rid)
    engine.cache.check_invariants()


def test_two_layers_of_the_1b_shape_in_mixed_steps_of_64_requests(capsys):
    """24 query heads on 8 kv heads of 64, hidden 1,536.  Up to 64 live requests; a step brings every decoding request's
    next token (about 50 rows) and up to two portions of at most 512 tokens of requests whose prompts are still being
    read; requests that end give their pages to the ones that join, and the pool holds no more than the live requests
    need.  The last row of every portion and every third decoded token's logits (the others' logits are not asked for:
    they still run, and what they leave in the cache is read by the steps after) are compared when a request ends."""
    rng = random.Random(9)
    V = SHAPE_1B["vocab_size"]
    n_total, n_decode, live_max = 100, 40, 64
    prompt = {("r%02d" % i): rng.randint(128, 1024) for i in range(n_total)}
    toks = {rid: H.random_tokens(V, n + n_decode, 400 + i) for i, (rid, n) in enumerate(prompt.items())}
    # the trace: every decoding request's token, up to two portions of 512, admissions first come first served
    pending, live, steps, peak = list(prompt), {}, [], 0
    while pending or live:
        while pending and len(live) < live_max:
            live[pending.pop(0)] = 0
        entries, portions = [], 0
        for rid in list(live):
            cur, n = live[rid], prompt[rid]
            if cur >= n:
                k = cur - n
                entries.append((rid, [toks[rid][cur]], [0] if (k % 3 == 0 or k == n_decode - 1) else []))
                live[rid] = cur + 1
            elif portions < 2:
                s = min(512, n - cur)
                entries.append((rid, toks[rid][cur:cur + s], [s - 1]))
                live[rid] = cur + s
                portions += 1
        peak = max(peak, sum(H.ceil64(c) for c in live.values() if c > 0))
        ends = [rid for rid in live if live[rid] == prompt[rid] + n_decode]
        for rid in ends:
            del live[rid]
        if entries:
            steps.append((entries, ends))
    engine, sd = _engine_and_weights(SHAPE_1B, seed=13, std=0.02, max_tokens=peak, max_requests=live_max)
    got, cursor, most_rows, seen_pages, worst, n_places = {}, {}, 0, {}, (0.0, None), 0
    for entries, ends in steps:
        out = _step(engine, entries)
        most_rows = max(most_rows, sum(1 for e in entries if len(e[1]) == 1))
        i = 0
        for rid, t, want in entries:
            base = cursor.get(rid, 0)
            for w in want:
                got.setdefault(rid, {})[base + w] = out[i].clone()
                i += 1
            cursor[rid] = base + len(t)
            for pg in engine.cache.block_table(rid, 0):
                seen_pages.setdefault(pg, set()).add(rid)
        for rid in ends:
            engine.free(rid)
            mine = got.pop(rid)
            ref = _plain_rows(SHAPE_1B, sd, toks[rid], list(mine))
            w = H.compare_places({(rid, p): r for p, r in mine.items()}, {(rid, p): r for p, r in ref.items()}, H.BF16_TOL,
                                 "1B shape, mixed steps")
            worst = max(worst, w, key=lambda x: x[0])
            n_places += len(mine)
    # many single tokens a step; pages served several requests in turn; every request was compared
    assert most_rows >= 45 and max(len(v) for v in seen_pages.values()) >= 2 and not got and n_places >= n_total * 14
    with capsys.disabled():
        print("\n1B shape (2 layers), %d steps, up to %d single tokens beside two portions, %d places: worst error %.3g at %s"
              % (len(steps), most_rows, n_places, worst[0], worst[1]))
    engine.cache.check_invariants()
    assert not engine.cache.requests
