#!/usr/bin/python3
"""Decode and prefill throughput of the MiniCPM-2B-shaped model on one MI355X.

  python bench.py --gpus 1 --steps K --warmup W

A step is one decode step of the whole batch: the scheduler's step (plan, the step
function over one new token per request, greedy sampling on the device, the sampled
tokens fed back and the finish rules checked); the reference times the same loop,
scripts/jiuge.py:562-583, prefill excluded.  Weights are random (seeded), prompts are
seeded uniform-random token ids.  One JSON line is printed.

  --workload mixed   the 1B shape's workload: 64 requests, prompts of 128..2,048 tokens, portions of 512
  --workload long    the 8B shape's workload: 4 prompts of 16,384 tokens, then decoding
  --direct           decode by calling the step function directly, without the scheduler
"""
import argparse
import json
import math
import os
import sys
import time

import torch

HBM_PEAK_GBS = 8000.0           # MI355X HBM3E
PEAK_TFLOPS = {"bf16": 2500.0, "fp32": 157.3}

# The benchmark's configuration: MiniCPM-2B-shaped (40 layers, hidden 2304, 36 heads of 64, vocabulary 122753)
MODEL = dict(
    model_type="minicpm", vocab_size=122753, hidden_size=2304, num_hidden_layers=40,
    num_attention_heads=36, num_key_value_heads=36, intermediate_size=5760,
    max_position_embeddings=4096, rms_norm_eps=1e-5, rope_theta=10000.0,
    scale_emb=12, dim_model_base=256, scale_depth=1.4, tie_word_embeddings=True, eos_token_id=2)
# Two further shapes for --shape: MiniCPM-1B-shaped (deep, narrow, 3 query heads per kv head) and
# MiniCPM4-8B/FM9G-8B-shaped (16 query heads per kv head, head size 128, longrope).  The default run is 2b.
def _seeded_factors(seed, n=64):
    """Long-context rotary factors drawn from the seed, uniform in [1, 4]."""
    import random
    rng = random.Random(seed)
    return [1.0 + 3.0 * rng.random() for _ in range(n)]


SHAPES = {
    "2b": MODEL,
    "1b": dict(MODEL, vocab_size=73440, hidden_size=1536, num_hidden_layers=52, num_attention_heads=24,
               num_key_value_heads=8, intermediate_size=3840),
    "8b": dict(MODEL, vocab_size=73448, hidden_size=4096, num_hidden_layers=32, num_attention_heads=32,
               num_key_value_heads=2, intermediate_size=16384, rms_norm_eps=1e-6, tie_word_embeddings=False,
               max_position_embeddings=32768,
               rope_scaling=dict(type="longrope", original_max_position_embeddings=32768,
                                 short_factor=_seeded_factors(1), long_factor=_seeded_factors(2))),
}
PROMPT = 2048
BATCH = 8
WEIGHT_STD = 0.1


def _sync():
    torch.cuda.synchronize()


DTYPE = torch.bfloat16          # --dtype float32: the whole model in true 32-bit (weights, activations, cache, products)


def _elem_bytes():
    return 2 if DTYPE == torch.bfloat16 else 4


def build_engine(layers, max_tokens, max_requests, page_size):
    from infinicore_infer_amd.config import config_from_dict
    from infinicore_infer_amd.engine import Engine
    from infinicore_infer_amd.parts import Runtime, build_model
    from infinicore_infer_amd.weights import init_random_weights
    cfg = dict(MODEL, num_hidden_layers=layers or MODEL["num_hidden_layers"])
    conf = config_from_dict(cfg)
    model = build_model(conf.model_spec(), Runtime(dtype=DTYPE, device="cuda:0"))
    init_random_weights(model, seed=0, std=WEIGHT_STD, tie=bool(cfg.get("tie_word_embeddings", True)))
    return Engine(model, max_tokens=max_tokens, page_size=page_size, max_requests=max_requests), conf


def model_numbers(conf):
    """Bytes of weights a decode step reads once, cache bytes per token, flops per prefill."""
    d, L, di, V = conf.hidden_size, conf.num_hidden_layers, conf.intermediate_size, conf.vocab_size
    nh, nkvh, dh = conf.num_attention_heads, conf.num_key_value_heads, conf.head_dim
    per_layer = (nh + 2 * nkvh) * dh * d + nh * dh * d + 3 * d * di
    eb = _elem_bytes()
    weight_bytes = eb * (L * per_layer + V * d) + 4 * d * (2 * L + 1)      # the head's table once; embedding rows are negligible
    kv_bytes_per_token = 2 * L * nkvh * dh * eb

    def prefill_flops(T):
        linear = 2.0 * T * L * per_layer
        attn = L * nh * dh * 4.0 * (T * (T + 1) / 2)        # QK^T and PV over the causal half
        head = 2.0 * V * d                                   # last row only
        return linear + attn + head
    return weight_bytes, kv_bytes_per_token, prefill_flops


def time_prefill(engine, tokens, reps=6):
    """Mean time of a whole-prompt step with its sampled token (one untimed pass first)."""
    from infinicore_infer_amd.engine import StepEntry
    total = 0.0
    for i in range(reps + 1):
        _sync()
        t0 = time.perf_counter()
        logits = engine.step([StepEntry("pf", tokens, [len(tokens) - 1])])
        engine.sample(logits)
        _sync()
        dt = time.perf_counter() - t0
        engine.free("pf")
        if i > 0:
            total += dt
    return total / reps


def time_decode_scheduled(engine, batch, steps, warmup, vocab, seed=0):
    """``batch`` requests of PROMPT tokens go through the scheduler; once all of them decode, ``warmup``
    untimed and ``steps`` timed steps (each: one token for every request)."""
    from infinicore_infer_amd.engine.scheduler import Scheduler
    from infinicore_infer_amd.engine.tasks import InferTask
    g = torch.Generator().manual_seed(seed)
    sch = Scheduler(engine, max_batch_tokens=max(PROMPT, batch), chunk_size=PROMPT, overlap=True)
    for i in range(batch):
        toks = torch.randint(0, vocab, (PROMPT,), generator=g).tolist()
        sch.add(InferTask("d%d" % i, toks, 1 << 30, temperature=0.0, topk=1, end_tokens=[],
                          max_new_tokens=warmup + steps + batch + 8))     # the first ones decode while the others' prompts run
    while sch.waiting or any(not r.decoding for r in sch.running):
        sch.step()
    # (decoding runs one step ahead of the host: a call issues at most one step and returns the tokens of the one before)
    first = sch.n_steps
    while sch.n_steps < first + warmup:
        sch.step()
    _sync()
    ctx0 = engine.length("d0")
    first = sch.n_steps
    t0 = time.perf_counter()
    while sch.n_steps < first + steps:
        sch.step()
    _sync()
    dt = time.perf_counter() - t0
    ctx1 = engine.length("d0")
    assert sch.n_steps == first + steps and ctx1 - ctx0 == steps
    assert len(sch.running) == batch and sch.n_preempted == 0
    for i in range(batch):
        sch.abort("d%d" % i)
    return dt / steps, (ctx0 + ctx1) / 2.0


def time_decode(engine, batch, steps, warmup, vocab, seed=0):
    """Prefill ``batch`` requests of PROMPT tokens, then time ``steps`` decode steps."""
    from infinicore_infer_amd.engine import StepEntry
    g = torch.Generator().manual_seed(seed)
    ids = ["d%d" % i for i in range(batch)]
    last = []
    for rid in ids:
        toks = torch.randint(0, vocab, (PROMPT,), generator=g).tolist()
        logits = engine.step([StepEntry(rid, toks, [PROMPT - 1])])
        last.append(engine.sample(logits)[0])

    def one():
        nonlocal last
        logits = engine.step([StepEntry(rid, [t], [0]) for rid, t in zip(ids, last)])
        last = engine.sample(logits)

    for _ in range(warmup):
        one()
    _sync()
    ctx0 = engine.length(ids[0])
    t0 = time.perf_counter()
    for _ in range(steps):
        one()
    _sync()
    dt = time.perf_counter() - t0
    ctx1 = engine.length(ids[0])
    for rid in ids:
        engine.free(rid)
    return dt / steps, (ctx0 + ctx1) / 2.0


def run_mixed(args):
    """The 1B-shaped configuration's workload: 64 requests with prompts of 128..2,048 tokens go through the
    scheduler, which cuts the prompts into portions of 512 under a token budget per step and decodes the
    running requests beside them.  One JSON line: all tokens (prompt and generated) per second."""
    import random
    from infinicore_infer_amd.engine.scheduler import Scheduler
    from infinicore_infer_amd.engine.tasks import InferTask
    n_req, gen, chunk, budget = args.requests, args.steps, 512, args.token_budget
    rnd = random.Random(0)
    lens = [rnd.randint(128, 2048) for _ in range(n_req)]
    pool = sum((l + gen + args.page_size - 1) // args.page_size * args.page_size for l in lens) + 64 * args.page_size
    engine, conf = build_engine(args.layers, pool, n_req, args.page_size)
    if not args.no_tune:
        # the two step sizes that recur: a full token budget, and one token of every request
        engine.tune_library_products([budget] + [b for b in (n_req,) if b > 16])
    g = torch.Generator().manual_seed(1)
    prompts = [torch.randint(0, conf.vocab_size, (l,), generator=g).tolist() for l in lens]

    def run():
        sch = Scheduler(engine, max_batch_tokens=budget, chunk_size=chunk, overlap=True)
        for i, toks in enumerate(prompts):
            sch.add(InferTask(i, toks, conf.max_position_embeddings, temperature=0.0, topk=1, end_tokens=[], max_new_tokens=gen))
        _sync()
        t0 = time.perf_counter()
        steps = []
        while sch.has_unfinished():
            s0, issued = time.perf_counter(), sch.n_steps
            sch.step()
            took = time.perf_counter() - s0
            if sch.n_steps > issued:                    # the call issued a step (while decoding runs ahead it also waited for the one before)
                steps.append((took, sum(n for _, _, n in sch.last_plan)))
            elif steps:                                 # it only read the tokens of the step in flight
                steps[-1] = (steps[-1][0] + took, steps[-1][1])
        _sync()
        return time.perf_counter() - t0, steps, sch.n_preempted

    run()                                            # one untimed pass: buffers grow, graphs are recorded
    dt, steps, preempted = run()
    total = sum(lens) + n_req * gen
    mixed = [s for s in steps if s[1] > n_req]
    dec = [s for s in steps if s[1] <= n_req]
    out = {
        "metric": "tokens/s (prompt + generated) through the scheduler, %d requests, prompts 128..2048, portions of %d "
                  "(MiniCPM-%s-shaped)" % (n_req, chunk, args.shape.upper()),
        "value": round(total / dt, 1), "unit": "tokens/s", "n_gpus": 1, "steps": len(steps), "warmup": 1,
        "ms_per_step": round(dt / len(steps) * 1e3, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic (seeded random weights N(0,0.1) and token ids)",
        "config": {
            "model": "MiniCPM-%s-shaped" % args.shape.upper(), "layers": conf.num_hidden_layers, "layers_of_config": MODEL["num_hidden_layers"],
            "hidden": conf.hidden_size, "heads": conf.num_attention_heads, "kv_heads": conf.num_key_value_heads,
            "head_dim": conf.head_dim, "intermediate": conf.intermediate_size, "vocab": conf.vocab_size,
            "requests": n_req, "prompt_tokens": sum(lens), "generated_each": gen, "token_budget": budget, "portion": chunk,
            "page_size": args.page_size, "parallelism": "single-gpu", "sampling": "greedy on device",
        },
        "mixed_steps": {"count": len(mixed), "mean_ms": round(1e3 * sum(s[0] for s in mixed) / max(1, len(mixed)), 3),
                        "mean_tokens": round(sum(s[1] for s in mixed) / max(1, len(mixed)), 1)},
        "decode_steps": {"count": len(dec), "mean_ms": round(1e3 * sum(s[0] for s in dec) / max(1, len(dec)), 3)},
        "preempted": preempted,
    }
    weight_bytes, kv_per_tok, prefill_flops = model_numbers(conf)
    if mixed:      # a mixed step's matrix-product flops (its prompt portions dominate) against the bf16 peak
        d, L, di = conf.hidden_size, conf.num_hidden_layers, conf.intermediate_size
        per_tok = 2.0 * L * ((conf.num_attention_heads + 2 * conf.num_key_value_heads) * conf.head_dim * d
                             + conf.num_attention_heads * conf.head_dim * d + 3 * d * di)
        t_mixed = sum(s[0] for s in mixed) / len(mixed)
        n_mixed = sum(s[1] for s in mixed) / len(mixed)
        out["prefill"] = {"value": round(n_mixed / t_mixed, 1), "tokens": round(n_mixed, 1), "ms": round(t_mixed * 1e3, 3),
                          "frac": round(per_tok * n_mixed / t_mixed / (PEAK_TFLOPS["bf16"] * 1e12), 4)}
    if dec:        # a decode-only step reads every weight once and the live requests' cache
        t_dec = sum(s[0] for s in dec) / len(dec)
        ctx_mean = sum(lens) / len(lens) + gen / 2.0
        achieved = (weight_bytes + n_req * ctx_mean * kv_per_tok) / t_dec / 1e9
        out["roofline"] = {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                           "frac": round(achieved / HBM_PEAK_GBS, 4)}
    print(json.dumps(out))
    return 0


def main():
    global BATCH, MODEL, PROMPT, DTYPE
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--layers", type=int, default=0, help="fewer layers than the shape has (0: all)")
    ap.add_argument("--shape", default=None, choices=sorted(SHAPES), help="2b is the benchmark's configuration (default; 1b for --workload mixed)")
    ap.add_argument("--workload", default="decode", choices=["decode", "mixed", "long"],
                    help="decode: the benchmark (prefill of one prompt, decode steps at fixed batches); "
                         "mixed: 64 requests of 128..2048 prompt tokens through the scheduler, --steps tokens generated each; "
                         "long: the 8B shape with 4 prompts of 16,384 tokens (the same as --shape 8b --prompt 16384 --batch 4 --no-points)")
    ap.add_argument("--direct", action="store_true", help="decode through the step function directly, not through the scheduler")
    ap.add_argument("--requests", type=int, default=64, help="--workload mixed: number of requests")
    ap.add_argument("--token-budget", type=int, default=1024, help="--workload mixed: tokens per step")
    ap.add_argument("--prompt", type=int, default=PROMPT)
    ap.add_argument("--page-size", type=int, default=64)
    ap.add_argument("--no-points", action="store_true", help="skip the batch 1 and 64 points")
    ap.add_argument("--no-tune", action="store_true", help="keep the library's default kernel choice for prefill products")
    ap.add_argument("--batch", type=int, default=BATCH, help="batch of the headline run (for profiling other points)")
    ap.add_argument("--eager", action="store_true", help="decode without HIP graphs (so that a profiler's counters attribute to kernels)")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"],
                    help="float32: the whole model in true 32-bit (no reduced-precision matrix mode), against the fp32 peak")
    args = ap.parse_args()
    DTYPE = {"bfloat16": torch.bfloat16, "float32": torch.float32}[args.dtype]
    dname = "bf16" if DTYPE == torch.bfloat16 else "fp32"
    if args.gpus != 1:
        print("bench.py: this engine runs on one GPU; --gpus %d is not supported" % args.gpus)
        return 2

    sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
    if args.workload == "long":
        args.shape = args.shape or "8b"
        if args.prompt == ap.get_default("prompt"):
            args.prompt = 16384
        if args.batch == ap.get_default("batch"):
            args.batch = 4
        args.no_points = True
    if args.shape is None:
        args.shape = "1b" if args.workload == "mixed" else "2b"
    MODEL, PROMPT = SHAPES[args.shape], args.prompt
    if args.workload == "mixed":
        if args.steps == ap.get_default("steps"):
            args.steps = 64
        return run_mixed(args)
    per_req = PROMPT + args.warmup + args.steps + 64 + max(BATCH, args.batch, 64)
    per_req = (per_req + 63) // 64 * 64
    BATCH = args.batch
    batches = [BATCH] if args.no_points else sorted({BATCH, 1, 64}, key=lambda b: (b != BATCH, b))
    engine, conf = build_engine(args.layers, per_req * max(batches), max(batches) + 1, args.page_size)
    weight_bytes, kv_per_tok, prefill_flops = model_numbers(conf)
    vocab = conf.vocab_size
    if args.eager:
        engine.use_graphs = False

    if not args.no_tune:
        # the library's algorithm choice for the products of the prefill and of decoding at batches beyond 16
        engine.tune_library_products([PROMPT] + [b for b in batches if b > 16])
    g = torch.Generator().manual_seed(123)
    ptoks = torch.randint(0, vocab, (PROMPT,), generator=g).tolist()
    t_pf = time_prefill(engine, ptoks)
    pf_flops = prefill_flops(PROMPT)

    results = {}
    decode = time_decode if args.direct else time_decode_scheduled
    for b in batches:
        results[b] = decode(engine, b, args.steps, args.warmup, vocab, seed=b)
    ms, ctx = results[BATCH][0] * 1e3, results[BATCH][1]
    value = BATCH / results[BATCH][0]
    bytes_step = weight_bytes + BATCH * ctx * kv_per_tok
    achieved = bytes_step / results[BATCH][0] / 1e9

    out = {
        "metric": "decode tokens/s, batch %d, %d-token prompts (MiniCPM-%s-shaped)" % (BATCH, PROMPT, args.shape.upper()),
        "value": round(value, 1), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": dname, "data": "synthetic (seeded random weights N(0,0.1) and token ids)",
        "config": {
            "model": "MiniCPM-%s-shaped" % args.shape.upper(), "layers": conf.num_hidden_layers, "layers_of_config": MODEL["num_hidden_layers"],
            "hidden": conf.hidden_size, "heads": conf.num_attention_heads, "kv_heads": conf.num_key_value_heads,
            "head_dim": conf.head_dim, "intermediate": conf.intermediate_size, "vocab": conf.vocab_size,
            "global_batch": BATCH, "seq_len": PROMPT, "context_mean": round(ctx, 1), "generated": args.steps,
            "page_size": args.page_size, "tied_embeddings": bool(MODEL.get("tie_word_embeddings", True)), "parallelism": "single-gpu",
            "sampling": "greedy on device", "library_gemm": "default" if args.no_tune else "algorithms timed per shape",
            "decode_launch": "eager" if args.eager else "hip graph", "decode_loop": "direct" if args.direct else "scheduler",
        },
        "prefill": {"value": round(PROMPT / t_pf, 1), "tokens": PROMPT, "ms": round(t_pf * 1e3, 3),
                    "frac": round(pf_flops / t_pf / (PEAK_TFLOPS[dname] * 1e12), 4)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4)},
        "points": {("decode_b%d" % b): round(b / results[b][0], 1) for b in batches if b != BATCH},
        # every point's step against the same bound: the bytes it has to read (weights once, the live requests' cache) / its time
        "points_roofline": {("decode_b%d" % b): {
            "ms": round(results[b][0] * 1e3, 4), "context": round(results[b][1], 1),
            "achieved": round((weight_bytes + b * results[b][1] * kv_per_tok) / results[b][0] / 1e9, 1),
            "frac": round((weight_bytes + b * results[b][1] * kv_per_tok) / results[b][0] / 1e9 / HBM_PEAK_GBS, 4)}
            for b in batches},
    }
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
