"""Trace replay: feed given token ids through the model step by step and write
the logits at the wanted places.  Nothing is sampled.  It drives the same
model, step function, cache and kernels that generation uses.

Input: one JSON object a line,
  {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}
Output: for a step in which something is wanted, ``<out>/<step>.f32``: the
logits at the wanted places in the order of the entries and of ``want``, as
little-endian float32 [wanted, vocab]; after every step a line ``done <step>``.
"""
import json
import os
import sys

import torch

from .engine import Engine, StepEntry

_DTYPES = {"bfloat16": torch.bfloat16, "float32": torch.float32}


def replay(engine: Engine, lines, out_dir: str, log=sys.stdout) -> int:
    os.makedirs(out_dir, exist_ok=True)
    n = 0
    for line in lines:
        line = line.strip()
        if not line:
            continue
        rec = json.loads(line)
        step = rec["step"]
        entries = [StepEntry(e["id"], e["tokens"], e.get("want", [])) for e in rec.get("entries", [])]
        logits = engine.step(entries) if entries else None
        if logits is not None:
            arr = logits.to(torch.float32).cpu().contiguous().numpy().astype("<f4", copy=False)
            tmp = os.path.join(out_dir, ".%s.f32.tmp" % step)
            with open(tmp, "wb") as f:
                f.write(arr.tobytes())
            os.replace(tmp, os.path.join(out_dir, "%s.f32" % step))
        for rid in rec.get("end", []):
            engine.free(rid)
        print("done %s" % step, file=log, flush=True)
        n += 1
    return n


def main(argv=None) -> int:
    import argparse
    ap = argparse.ArgumentParser(prog="trace_run", description="replay a token trace through the engine")
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", required=True, choices=sorted(_DTYPES))
    ap.add_argument("--out", required=True, help="folder for <step>.f32 files")
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="most tokens live requests hold at any time (each rounded up to 64)")
    ap.add_argument("--page-size", type=int, default=16, choices=(16, 32, 64))
    ap.add_argument("--device", default="cuda:0")
    ap.add_argument("--attention", default="auto", choices=("auto", "generic"))
    args = ap.parse_args(argv)

    print("[trace_run] loading kernels and model from %s (%s)" % (args.model, args.dtype),
          file=sys.stderr, flush=True)
    engine = Engine.from_dir(args.model, dtype=_DTYPES[args.dtype], device=args.device,
                             max_tokens=args.max_tokens, page_size=args.page_size, max_requests=64,
                             attention_impl=args.attention)
    print("[trace_run] ready", file=sys.stderr, flush=True)
    replay(engine, sys.stdin, args.out)
    torch.cuda.synchronize()
    return 0


if __name__ == "__main__":
    sys.exit(main())
