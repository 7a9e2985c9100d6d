"""Shared by the tests: the two tiny configurations, model folders in temporary
directories, traces in the four replay modes, and the comparison rule."""
import json
import math
import os
import random

import torch

# Tolerances, fixed before the first GPU run and never widened: the largest
# absolute logit difference allowed, as a fraction of the largest |reference logit|.
FP32_TOL = 1e-4
BF16_TOL = 2e-2

# Tiny A: GQA 2:1, tied, muP constants != 1, head size 16, unit norm weights.
TINY_A = dict(
    model_type="minicpm", architectures=["MiniCPMForCausalLM"],
    vocab_size=256, hidden_size=64, num_hidden_layers=2, num_attention_heads=4, num_key_value_heads=2,
    intermediate_size=160, max_position_embeddings=128, rms_norm_eps=1e-5, rope_theta=10000.0,
    scale_emb=12, dim_model_base=16, scale_depth=1.4, tie_word_embeddings=True, eos_token_id=2)
TINY_A_INIT = dict(std=0.02, norm_std=0.0)

# Tiny B: every size and option differs: MHA, untied, neutral muP constants, head size 32,
# odd vocabulary, three layers, random norm weights, other theta and eps.
TINY_B = dict(
    model_type="fm9g", architectures=["FM9GForCausalLM"],
    vocab_size=509, hidden_size=96, num_hidden_layers=3, num_attention_heads=3, num_key_value_heads=3,
    intermediate_size=256, max_position_embeddings=256, rms_norm_eps=1e-6, rope_theta=1000000.0,
    scale_emb=1.0, dim_model_base=96, scale_depth=1.0, tie_word_embeddings=False, eos_token_id=[1, 3])
TINY_B_INIT = dict(std=0.05, norm_std=0.1)

# Tiny C: head size 64 (the tiled attention kernels), GQA 3:1, longrope, width and vocabulary
# that are no power of two.
TINY_C = dict(
    model_type="minicpm", vocab_size=331, hidden_size=200, num_hidden_layers=2, num_attention_heads=6,
    num_key_value_heads=2, head_dim=64, intermediate_size=344, max_position_embeddings=512,
    rms_norm_eps=1e-5, rope_theta=10000.0, scale_emb=4.0, dim_model_base=50, scale_depth=2.0,
    tie_word_embeddings=False, eos_token_id=2,
    rope_scaling=dict(type="longrope", original_max_position_embeddings=128,
                      short_factor=[1.0 + 0.05 * i for i in range(32)],
                      long_factor=[1.0 + 0.09 * i for i in range(32)]))
TINY_C_INIT = dict(std=0.05, norm_std=0.1)

# Tiny D: head size 128, four query heads on one kv head, hidden size below heads x head size.
TINY_D = dict(
    model_type="fm9g", vocab_size=300, hidden_size=136, num_hidden_layers=2, num_attention_heads=4,
    num_key_value_heads=1, head_dim=128, intermediate_size=200, max_position_embeddings=384,
    rms_norm_eps=1e-6, rope_theta=50000.0, scale_emb=2.0, dim_model_base=34, scale_depth=1.0,
    tie_word_embeddings=True, eos_token_id=[])
TINY_D_INIT = dict(std=0.06, norm_std=0.05)

CONFIGS = {"A": (TINY_A, TINY_A_INIT), "B": (TINY_B, TINY_B_INIT), "C": (TINY_C, TINY_C_INIT),
           "D": (TINY_D, TINY_D_INIT)}


def make_model_dir(tmp_path, name, seed=0, dtype=torch.bfloat16):
    from infinicore_infer_amd.weights import write_random_model
    cfg, init = CONFIGS[name]
    folder = os.path.join(str(tmp_path), "model_%s_%d_%s" % (name, seed, str(dtype).split(".")[-1]))
    if not os.path.isdir(folder):
        write_random_model(folder, cfg, seed=seed, dtype=dtype, **init)
    return folder


def load_state_dict(folder):
    from safetensors.torch import load_file
    return load_file(os.path.join(folder, "model.safetensors"))


def random_tokens(vocab, n, seed):
    rng = random.Random(seed)
    return [rng.randrange(vocab) for _ in range(n)]


def ceil64(n):
    return (n + 63) // 64 * 64


# ---------------------------------------------------------------------------
# traces
# ---------------------------------------------------------------------------
def trace_whole(requests):
    """Each request alone and whole, every position wanted."""
    steps = []
    for i, (rid, toks) in enumerate(requests.items()):
        steps.append({"step": i, "entries": [{"id": rid, "tokens": toks, "want": list(range(len(toks)))}],
                      "end": [rid]})
    return steps, max(ceil64(len(t)) for t in requests.values())


def trace_last_one_by_one(requests, tail=32):
    """Most of a request in one step, the last ``tail`` tokens one by one."""
    steps, n = [], 0
    for rid, toks in requests.items():
        head = max(1, len(toks) - tail) if len(toks) > tail else 1
        steps.append({"step": n, "entries": [{"id": rid, "tokens": toks[:head], "want": list(range(head))}], "end": []})
        n += 1
        for j in range(head, len(toks)):
            steps.append({"step": n, "entries": [{"id": rid, "tokens": [toks[j]], "want": [0]}],
                          "end": [rid] if j == len(toks) - 1 else []})
            n += 1
        if head == len(toks):
            steps[-1]["end"] = [rid]
    return steps, max(ceil64(len(t)) for t in requests.values())


def trace_chunks(requests, sizes=(16, 5, 2, 9, 3, 2, 31, 2, 7)):
    """Portions of changing size, down to two tokens."""
    steps, n, k = [], 0, 0
    for rid, toks in requests.items():
        pos = 0
        while pos < len(toks):
            s = min(sizes[k % len(sizes)], len(toks) - pos)
            k += 1
            last = pos + s == len(toks)
            steps.append({"step": n, "entries": [{"id": rid, "tokens": toks[pos:pos + s], "want": list(range(s))}],
                          "end": [rid] if last else []})
            n += 1
            pos += s
    return steps, max(ceil64(len(t)) for t in requests.values())


def trace_mixed(requests, live_max=4, sizes=(7, 2, 16, 3, 11, 2, 29, 5), tail=6, seed=0):
    """Up to ``live_max`` live requests; portions of some beside single tokens of
    others; a request is sometimes left out of a step; requests end while others
    go on, so their pages are handed to the next ones.  Returns the steps and the
    smallest --max-tokens that holds the live requests at every time."""
    rng = random.Random(seed)
    pending = list(requests.items())
    live = {}            # id -> cursor
    steps, n, k = [], 0, 0
    peak = 0
    while pending or live:
        while pending and len(live) < live_max:
            rid, _ = pending.pop(0)
            live[rid] = 0
        entries, ends = [], []
        ids = list(live)
        for rid in ids:
            toks = requests[rid]
            cur = live[rid]
            if len(ids) > 1 and rng.random() < 0.2:
                continue                       # left out of this step
            if len(toks) - cur <= tail:
                s = 1                          # the tail is fed token by token
            else:
                s = min(sizes[k % len(sizes)], len(toks) - tail - cur)
                k += 1
            entries.append({"id": rid, "tokens": toks[cur:cur + s], "want": list(range(s))})
            live[rid] = cur + s
        peak = max(peak, sum(ceil64(c) for c in live.values() if c > 0))
        for rid in ids:
            if live[rid] == len(requests[rid]):
                ends.append(rid)
                del live[rid]
        if entries:
            steps.append({"step": n, "entries": entries, "end": ends})
            n += 1
    return steps, peak


def wanted_places(steps):
    """The set of (id, position) whose logits a trace asks for."""
    places, cursor = set(), {}
    for rec in steps:
        for e in rec["entries"]:
            base = cursor.get(e["id"], 0)
            places.update((e["id"], base + w) for w in e["want"])
            cursor[e["id"]] = base + len(e["tokens"])
        for rid in rec["end"]:
            cursor.pop(rid, None)
    return places


def run_trace(engine, steps):
    """Feed steps to the engine; returns {(id, position): float32 logits row (CPU)}.  A step must return exactly
    one row for every place it wants: a step that returns nothing, or too few rows, fails here."""
    from infinicore_infer_amd.engine import StepEntry
    got = {}
    cursor = {}
    for rec in steps:
        entries = [StepEntry(e["id"], e["tokens"], e["want"]) for e in rec["entries"]]
        logits = engine.step(entries)
        n_wanted = sum(len(e["want"]) for e in rec["entries"])
        if n_wanted == 0:
            assert logits is None, "step %s wants nothing and got logits" % rec.get("step")
        else:
            assert logits is not None, "step %s wants %d rows and got none" % (rec.get("step"), n_wanted)
            assert logits.shape[0] == n_wanted, "step %s wants %d rows and got %d" % (rec.get("step"), n_wanted, logits.shape[0])
            rows = logits.float().cpu()
            i = 0
            for e in rec["entries"]:
                base = cursor.get(e["id"], 0)
                for w in e["want"]:
                    got[(e["id"], base + w)] = rows[i].clone()
                    i += 1
        for e in rec["entries"]:
            cursor[e["id"]] = cursor.get(e["id"], 0) + len(e["tokens"])
        for rid in rec["end"]:
            engine.free(rid)
            cursor.pop(rid, None)
    return got


def plain_logits(cfg, sd, requests, bf16):
    from plain_model import plain_forward, round_bf16
    return {rid: plain_forward(cfg, sd, toks, rnd=round_bf16 if bf16 else None)
            for rid, toks in requests.items()}


def compare(got, ref, tol, what="", steps=None):
    """Every wanted row against the plain logits; reports the first wrong place.  ``got`` must hold rows (with
    ``steps`` given: exactly the places the trace wants), so a run that returned nothing cannot pass."""
    assert len(got) > 0, "%s: no logits to compare" % what
    if steps is not None:
        want = wanted_places(steps)
        assert set(got) == want, ("%s: %d of %d wanted places came back (missing e.g. %s)"
                                  % (what, len(set(got) & want), len(want), sorted(want - set(got), key=str)[:3]))
    worst, worst_at = 0.0, None
    for (rid, pos), row in sorted(got.items(), key=lambda kv: (str(kv[0][0]), kv[0][1])):
        r = ref[rid][pos]
        scale = float(ref[rid].abs().max())
        err = float((row.double() - r).abs().max()) / scale
        assert math.isfinite(err), "%s: non-finite logits at request %s position %d" % (what, rid, pos)
        if err > worst:
            worst, worst_at = err, (rid, pos)
        assert err <= tol, ("%s: request %s position %d differs by %.3g of the largest logit (allowed %.3g)"
                            % (what, rid, pos, err, tol))
    return worst, worst_at


def compare_places(got, ref, tol, what=""):
    """As ``compare`` for runs where only some positions were computed: ``ref`` maps (id, position) to the plain
    logits row.  Every place of ``ref`` must be in ``got`` and nothing else; the error is taken as a fraction of the
    largest plain logit of the request's rows."""
    assert len(got) > 0 and set(got) == set(ref), ("%s: wanted %d places, got %d (missing e.g. %s)"
                                                   % (what, len(ref), len(got), sorted(set(ref) - set(got), key=str)[:3]))
    scale = {}
    for (rid, _), r in ref.items():
        scale[rid] = max(scale.get(rid, 0.0), float(r.abs().max()))
    worst, worst_at = 0.0, None
    for key in sorted(got, key=lambda k: (str(k[0]), k[1])):
        err = float((got[key].double() - ref[key].double().cpu()).abs().max()) / scale[key[0]]
        assert math.isfinite(err), "%s: non-finite logits at request %s position %d" % (what, key[0], key[1])
        if err > worst:
            worst, worst_at = err, key
        assert err <= tol, ("%s: request %s position %d differs by %.3g of the largest logit (allowed %.3g)"
                            % (what, key[0], key[1], err, tol))
    return worst, worst_at
