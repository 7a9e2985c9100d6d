"""Python entry point and command line, in the manner of the reference's
scripts/jiuge.py, for any registered architecture.

    python -m infinicore_infer_amd.causal_lm --amd <path/to/model_dir> [n_device] [options]
    python -m infinicore_infer_amd.causal_lm --amd --random-weights --config <config.json> [options]

(``infinicore_infer_amd.minicpm`` is the same module's class and command line under the
architecture's name, as the reference names its script after its model.)

``CausalLM(model_dir_path, device, ndev, max_tokens)`` offers what
JiugeForCauslLM does (scripts/jiuge.py:396-643): ``max_context_len``,
``create_kv_cache`` / ``drop_kv_cache``, ``batch_infer_one_round(tasks)``,
``generate(input_content, max_steps, topp_, topk_, temperature_)``,
``perplexity(test_sequences, batch_size)`` and ``destroy_model_instance``.
The model is built from config.json through the architecture registry: nothing
here names an architecture.  The cache is paged, and there is one device kind.  Generation has one loop: the
scheduler's; ``generate`` and the command line hand it their requests.
"""
import math
import os
import sys
import time
from typing import List, Optional, Sequence

import torch

from .config import config_from_dir
from .engine import Engine, StepEntry
from .engine.scheduler import Scheduler
from .engine.tasks import InferTask, KVCache
from .sampling import uniform_draw

DEVICE_FLAGS = ("--amd", "--hip", "--mi355x")
_DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float32": torch.float32, "fp32": torch.float32}


class CausalLM:
    def __init__(self, model_dir_path, device="cuda:0", ndev=1, max_tokens=None, dtype=None,
                 cache_tokens: Optional[int] = None, page_size: int = 64, max_requests: int = 64,
                 prefix_cache: bool = False):
        """``max_tokens`` caps the context length as in the reference
        (scripts/jiuge.py:128-130); ``cache_tokens`` sizes the page pool (default:
        four full contexts); ``dtype`` None takes the checkpoint's torch_dtype; ``prefix_cache``
        keeps finished requests' caches so that later prompts go on from a shared prefix, as the
        reference's server pool does (scripts/kvcache_pool.py)."""
        if ndev != 1:
            raise ValueError("this engine runs on one GPU (ndev=%r)" % (ndev,))
        print("Loading model weights to host...")
        t0 = time.time()
        self.config = config_from_dir(model_dir_path, max_tokens=max_tokens)
        self.eos_token_id = list(self.config.eos_token_id)
        ctx = self.config.max_positions
        self.engine = Engine.from_dir(model_dir_path, dtype=dtype, device=device, max_context=max_tokens,
                                      max_tokens=cache_tokens or 4 * ctx, page_size=page_size,
                                      max_requests=max_requests)
        self.tokenizer = self._load_tokenizer(model_dir_path)
        self.prefix_cache = bool(prefix_cache)
        self._scheduler = None                  # kept between calls when finished requests' caches are kept
        print(f"Time used: {time.time() - t0:.3f}s")

    @staticmethod
    def _load_tokenizer(model_dir_path):
        """A tokenizer when the folder has one; token-id prompts need none."""
        if not any(os.path.isfile(os.path.join(model_dir_path, f))
                   for f in ("tokenizer.json", "tokenizer.model", "tokenizer_config.json")):
            return None
        try:
            from transformers import AutoTokenizer
            return AutoTokenizer.from_pretrained(model_dir_path, trust_remote_code=False)
        except Exception as e:                      # noqa: BLE001
            print("no tokenizer loaded (%s); prompts must be token ids" % e)
            return None

    # ---- the reference's surface --------------------------------------------------------
    def max_context_len(self):
        return self.config.max_positions

    def create_kv_cache(self):
        return KVCache(self)

    def drop_kv_cache(self, kv_cache):
        kv_cache.drop(self)

    def duplicate_kv_cache(self, kv_cache, seq_len: Optional[int] = None):
        """A second cache holding a copy of the first ``seq_len`` tokens of ``kv_cache``
        (duplicateKVCache, include/infinicore_infer/models/jiuge.h:66-69)."""
        new = KVCache(self)
        self.engine.fork(kv_cache.data(), new.data(), seq_len)
        new.tokens = list(kv_cache.tokens[:self.engine.length(new.data())])
        return new

    def batch_infer_one_round(self, tasks: List[InferTask]):
        """One step over the tasks' pending tokens; one sampled token per task
        (scripts/jiuge.py:529-537)."""
        entries = [StepEntry(t.kvcache().data(), t.tokens, [len(t.tokens) - 1]) for t in tasks]
        logits = self.engine.step(entries)
        if all(t.temperature == 0 or t.topk == 1 for t in tasks):
            return self.engine.sample(logits)
        return self.engine.sample(
            logits, [t.temperature for t in tasks], [t.topk for t in tasks], [t.topp for t in tasks],
            [uniform_draw(t.seed, t.id, len(t.generated)) for t in tasks])

    def encode(self, input_content):
        if isinstance(input_content, (list, tuple)):
            return [int(t) for t in input_content]
        if self.tokenizer is None:
            raise ValueError("the model folder has no tokenizer: give the prompt as a list of token ids")
        try:
            text = self.tokenizer.apply_chat_template(
                conversation=[{"role": "user", "content": input_content}],
                add_generation_prompt=True, tokenize=False)
        except Exception:                           # noqa: BLE001
            text = input_content
        print(text, end="", flush=True)
        return self.tokenizer.encode(text)

    def decode_token(self, token):
        if self.tokenizer is None:
            return "%d " % token
        return self.tokenizer.decode([token])

    def generate(self, input_content, max_steps, topp_=1.0, topk_=1, temperature_=1.0, seed=0,
                 max_batch_tokens=2048, chunk_size=512):
        """Generate up to ``max_steps`` tokens for one prompt (text, or a list of token
        ids); prints them as they come and returns (output, mean ms per step without the
        first token's), the surface of scripts/jiuge.py:539-586.  The request runs through the
        scheduler like any other (what the reference's server loop does for its tasks,
        scripts/launch_server.py:134-159): its prompt in portions, then token by token."""
        tokens = self.encode(input_content)
        pieces, step_times = [], []

        def on_step(new, seconds):
            for _task, tok in new:
                piece = self.decode_token(tok)
                pieces.append(piece)
                print(piece, end="", flush=True)
                step_times.append(seconds)

        outs = self._run_requests([tokens], max_steps, topp_, topk_, temperature_, seed, max_batch_tokens,
                                  chunk_size, on_step)
        print("\n")
        later = step_times[1:]
        avg_time = sum(later) * 1000 / max(len(later), 1)
        print(f"Time per step: {avg_time:.3f}ms")
        self.last_output_tokens = outs[0]
        return "".join(pieces), avg_time

    def generate_batch(self, prompts: Sequence[Sequence[int]], max_new_tokens, topp_=1.0, topk_=1,
                       temperature_=1.0, seed=0, max_batch_tokens=2048, chunk_size=512, on_step=None):
        """Several prompts through the scheduler (continuous batching, chunked prompts)."""
        return self._run_requests([list(p) for p in prompts], max_new_tokens, topp_, topk_, temperature_, seed,
                                  max_batch_tokens, chunk_size, on_step)

    def _run_requests(self, prompts, max_new_tokens, topp_, topk_, temperature_, seed, max_batch_tokens,
                      chunk_size, on_step=None):
        """The one generation loop: every request is a task of the scheduler."""
        if self.prefix_cache:                   # one scheduler for the model's life: it holds the kept caches
            if self._scheduler is None:
                self._scheduler = Scheduler(self.engine, max_batch_tokens=max_batch_tokens, chunk_size=chunk_size,
                                            prefix_cache=True)
            sched = self._scheduler
            sched.max_batch_tokens, sched.chunk_size = max_batch_tokens, chunk_size
        else:
            sched = Scheduler(self.engine, max_batch_tokens=max_batch_tokens, chunk_size=chunk_size, overlap=True)
        tasks = [InferTask("g%d" % i, list(p), self.max_context_len(), temperature_, topk_, topp_,
                           self.eos_token_id, seed=seed, max_new_tokens=max_new_tokens)
                 for i, p in enumerate(prompts)]
        for t in tasks:
            sched.add(t)
        sched.run(on_step)
        self.last_scheduler = sched
        self.last_tasks = tasks
        return [t.generated for t in tasks]

    def perplexity(self, test_sequences: List[Sequence[int]], batch_size=10):
        """exp(mean negative log-likelihood) of the sequences' next tokens, from the logits
        of all positions, log-softmax in float32 (scripts/jiuge.py:588-639)."""
        nll, total = 0.0, 0
        for i in range(0, len(test_sequences), batch_size):
            group = test_sequences[i:i + batch_size]
            entries, targets = [], []
            for j, seq in enumerate(group):
                inp = list(seq[:-1])
                entries.append(StepEntry("ppl%d" % j, inp, list(range(len(inp)))))
                targets.extend(seq[1:])
            logits = self.engine.step(entries).float()
            for e in entries:
                self.engine.free(e.req_id)
            logp = torch.log_softmax(logits, dim=-1)
            idx = torch.tensor(targets, dtype=torch.long, device=logp.device)
            nll += -float(logp[torch.arange(len(targets), device=logp.device), idx].sum())
            total += len(targets)
        return math.exp(nll / total)

    def destroy_model_instance(self):
        if self._scheduler is not None:
            self._scheduler.release_idle()
        self._scheduler = None
        self.engine = None
        torch.cuda.empty_cache()
        print("Model destroyed")



USAGE = ("Usage: python -m infinicore_infer_amd.causal_lm [--amd] <path/to/model_dir> [n_device] [options]\n"
         "   or: python -m infinicore_infer_amd.causal_lm [--amd] --random-weights --config <config.json> [options]\n"
         "options: [--device cuda:0] [--dtype bfloat16|float32] [--max-tokens N] [--prompt TEXT | --prompt-ids 1,2,3 ... | "
         "--prompt-len N [--num-prompts K]] [--max-new-tokens N] [--temperature T] [--top-k K] [--top-p P] [--seed S] "
         "[--page-size 16|32|64] [--num-pages N | --cache-tokens N] [--max-batch-tokens N] [--chunk-size N] "
         "[--prefix-cache] [--weights-seed S] [--weights-std X] [--weights-norm-std X]")

_OTHER_DEVICES = ("--cpu", "--nvidia", "--cambricon", "--ascend", "--metax", "--moore", "--iluvatar")


def _parse(argv):
    import argparse
    argv = list(argv)
    if argv and argv[0] in DEVICE_FLAGS:
        argv = argv[1:]
    elif argv and argv[0] in _OTHER_DEVICES:
        print("this engine runs on AMD MI355X only; use --amd")
        print(USAGE)
        sys.exit(1)
    model_path, ndev = None, 1
    if argv and not argv[0].startswith("--"):
        model_path = argv.pop(0)
        if argv and not argv[0].startswith("--"):
            ndev = int(argv.pop(0))
    ap = argparse.ArgumentParser(usage=USAGE)
    ap.add_argument("--random-weights", action="store_true",
                    help="no model folder: draw weights for --config from --weights-seed into a temporary folder")
    ap.add_argument("--config", default=None, help="a config.json of the architecture (with --random-weights)")
    ap.add_argument("--weights-seed", type=int, default=0)
    ap.add_argument("--weights-std", type=float, default=0.02)
    ap.add_argument("--weights-norm-std", type=float, default=0.0, help="norm weights are 1 + N(0, this)")
    ap.add_argument("--device", default="cuda:0")
    ap.add_argument("--dtype", default=None, choices=sorted(_DTYPES), help="default: the checkpoint's torch_dtype")
    ap.add_argument("--max-tokens", type=int, default=None, help="cap on a request's context (default: the model's)")
    ap.add_argument("--prompt", default=None, help="a text prompt (needs a tokenizer in the model folder)")
    ap.add_argument("--prompt-ids", action="append", default=None,
                    help="a prompt as comma-separated token ids; may be given several times")
    ap.add_argument("--prompt-len", type=int, default=None, help="random token ids of this length as the prompt (the first is bos_token_id if the configuration has one)")
    ap.add_argument("--num-prompts", type=int, default=1, help="with --prompt-len: how many such prompts")
    ap.add_argument("--max-new-tokens", "--max-steps", dest="max_new_tokens", type=int, default=500)
    ap.add_argument("--temperature", type=float, default=1.0)
    ap.add_argument("--top-k", "--topk", dest="topk", type=int, default=1)
    ap.add_argument("--top-p", "--topp", dest="topp", type=float, default=1.0)
    ap.add_argument("--seed", type=int, default=0, help="seed of the sampling draws (and of --prompt-len's tokens)")
    ap.add_argument("--page-size", type=int, default=64, choices=(16, 32, 64), help="tokens per cache page")
    ap.add_argument("--num-pages", type=int, default=None, help="pages of the cache pool")
    ap.add_argument("--cache-tokens", type=int, default=None, help="tokens the page pool holds (default: four contexts)")
    ap.add_argument("--max-batch-tokens", type=int, default=2048, help="tokens per step over all requests")
    ap.add_argument("--chunk-size", type=int, default=512, help="largest portion of a prompt per step")
    ap.add_argument("--prefix-cache", action="store_true",
                    help="keep finished requests' caches; later prompts go on from a shared prefix")
    args = ap.parse_args(argv)
    if (model_path is None) == (not args.random_weights):
        print("give a model folder, or --random-weights --config <config.json>")
        print(USAGE)
        sys.exit(1)
    if args.random_weights and not args.config:
        print("--random-weights needs --config <config.json>")
        sys.exit(1)
    if not str(args.device).startswith(("cuda", "hip")):
        print("this engine runs on the GPU only (--device %s)" % args.device)
        sys.exit(1)
    args.device = str(args.device).replace("hip", "cuda")
    return model_path, ndev, args


def test(argv=None):
    """The command line, in the manner of scripts/jiuge.py:646-677: a model folder, a prompt, tokens
    printed as they come and the time per step.  Several prompts run together through the scheduler."""
    import json
    import random
    import tempfile
    model_path, ndev, args = _parse(sys.argv[1:] if argv is None else argv)
    tmp = None
    if args.random_weights:
        from .weights import write_random_model
        with open(args.config, encoding="utf-8") as f:
            config = json.load(f)
        tmp = tempfile.TemporaryDirectory(prefix="infinicore_infer_amd_random_")
        model_path = write_random_model(tmp.name, config, args.weights_seed, std=args.weights_std,
                                        norm_std=args.weights_norm_std)
    cache_tokens = args.cache_tokens
    if args.num_pages is not None:
        cache_tokens = args.num_pages * args.page_size
    model = CausalLM(model_path, args.device, ndev, max_tokens=args.max_tokens,
                               dtype=_DTYPES[args.dtype] if args.dtype else None,
                               cache_tokens=cache_tokens, page_size=args.page_size, prefix_cache=args.prefix_cache)
    if args.prompt_ids:
        prompts = [[int(t) for t in p.split(",") if t.strip()] for p in args.prompt_ids]
    elif args.prompt_len:
        # as a tokenizer would: the configuration's bos token first, when it names one
        rng = random.Random(args.seed)
        bos = getattr(model.config, "bos_token_id", None)
        head = [int(bos)] if isinstance(bos, int) and 0 <= bos < model.config.vocab_size else []
        prompts = [(head + [rng.randrange(model.config.vocab_size) for _ in range(args.prompt_len)])[:args.prompt_len]
                   for _ in range(args.num_prompts)]
    else:
        prompts = [args.prompt if args.prompt is not None else "山东最高的山是？"]
    kw = dict(topp_=args.topp, topk_=args.topk, temperature_=args.temperature, seed=args.seed,
              max_batch_tokens=args.max_batch_tokens, chunk_size=args.chunk_size)
    if len(prompts) == 1:
        model.generate(prompts[0], args.max_new_tokens, **kw)
        outs = [model.last_output_tokens]
    else:
        t0 = time.time()
        outs = model.generate_batch(prompts, args.max_new_tokens, **kw)
        dt = time.time() - t0
        n = sum(len(o) for o in outs)
        print("%d requests, %d tokens generated in %.3f s (%.1f tokens/s), %d steps, %d preempted"
              % (len(prompts), n, dt, n / max(dt, 1e-9), model.last_scheduler.n_steps, model.last_scheduler.n_preempted))
    for i, (o, t) in enumerate(zip(outs, model.last_tasks)):
        print("tokens[%d] (%s): %s" % (i, t.finish_reason, " ".join(str(x) for x in o)))
    model.destroy_model_instance()
    if tmp is not None:
        tmp.cleanup()


if __name__ == "__main__":
    test()
