"""Python entry point and command line, in the manner of the reference's
scripts/jiuge.py.

    python -m infinicore_infer_amd.minicpm --amd <path/to/model_dir> [n_device] [options]

``MiniCPMForCausalLM(model_dir_path, device, ndev, max_tokens)`` offers what
JiugeForCauslLM does (scripts/jiuge.py:396-643): ``max_context_len``,
``create_kv_cache`` / ``drop_kv_cache``, ``batch_infer_one_round(tasks)``,
``generate(input_content, max_steps, topp_, topk_, temperature_)``,
``perplexity(test_sequences, batch_size)`` and ``destroy_model_instance``.
The model class is chosen from config.json through the architecture registry,
the cache is paged, and there is one device kind.
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


class MiniCPMForCausalLM:
    def __init__(self, model_dir_path, device="cuda:0", ndev=1, max_tokens=None, dtype=torch.bfloat16,
                 cache_tokens: Optional[int] = None, page_size: int = 64, max_requests: int = 64):
        """``max_tokens`` caps the context length as in the reference
        (scripts/jiuge.py:128-130); ``cache_tokens`` sizes the page pool (default:
        four full contexts)."""
        if ndev != 1:
            raise ValueError("this engine runs on one GPU (ndev=%r)" % (ndev,))
        print("Loading model weights to host...")
        t0 = time.time()
        self.config = config_from_dir(model_dir_path, max_tokens=max_tokens)
        self.eos_token_id = list(self.config.eos_token_id)
        ctx = self.config.max_position_embeddings
        self.engine = Engine.from_dir(model_dir_path, dtype=dtype, device=device, max_context=max_tokens,
                                      max_tokens=cache_tokens or 4 * ctx, page_size=page_size,
                                      max_requests=max_requests)
        self.tokenizer = self._load_tokenizer(model_dir_path)
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
        return self.config.max_position_embeddings

    def create_kv_cache(self):
        return KVCache(self)

    def drop_kv_cache(self, kv_cache):
        kv_cache.drop(self)

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

    def generate(self, input_content, max_steps, topp_=1.0, topk_=1, temperature_=1.0, seed=0):
        """Generate up to ``max_steps`` tokens for one prompt (text, or a list of token
        ids); prints them as they come and returns (output, mean ms per step without the
        first step), as scripts/jiuge.py:539-586 does."""
        tokens = self.encode(input_content)
        task = InferTask(0, tokens, self.max_context_len(), temperature_, topk_, topp_, self.eos_token_id,
                         seed=seed)
        task.bind_kvcache(KVCache(self))
        steps, total_time = 0, 0.0
        output_content = ""
        output_tokens = []
        for step_i in range(max_steps):
            start = time.time()
            out = self.batch_infer_one_round([task])[0]
            end = time.time()
            steps += 1
            piece = self.decode_token(out)
            output_content += piece
            output_tokens.append(out)
            print(piece, end="", flush=True)
            if out in self.eos_token_id:
                break
            task.next(out)
            if task.finish_reason is not None:
                break
            if step_i > 0:
                total_time += end - start
        print("\n")
        avg_time = total_time * 1000 / max(steps - 1, 1)
        print(f"Time per step: {avg_time:.3f}ms")
        task.kvcache().drop(self)
        self.last_output_tokens = output_tokens
        return output_content, avg_time

    def generate_batch(self, prompts: Sequence[Sequence[int]], max_new_tokens, topp_=1.0, topk_=1,
                       temperature_=1.0, seed=0, max_batch_tokens=2048, chunk_size=512):
        """Several prompts through the scheduler (continuous batching, chunked prompts)."""
        sched = Scheduler(self.engine, max_batch_tokens=max_batch_tokens, chunk_size=chunk_size)
        tasks = [InferTask("g%d" % i, list(p), self.max_context_len(), temperature_, topk_, topp_,
                           self.eos_token_id, seed=seed, max_new_tokens=max_new_tokens)
                 for i, p in enumerate(prompts)]
        for t in tasks:
            sched.add(t)
        sched.run()
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
        self.engine = None
        torch.cuda.empty_cache()
        print("Model destroyed")


USAGE = ("Usage: python -m infinicore_infer_amd.minicpm [--amd] <path/to/model_dir> [n_device] "
         "[--dtype bfloat16|float32] [--max-tokens N] [--prompt TEXT | --prompt-ids 1,2,3] [--max-steps N] "
         "[--temperature T] [--topk K] [--topp P] [--seed S] [--page-size 16|32|64] [--cache-tokens N]")


def test(argv=None):
    argv = list(sys.argv[1:] if argv is None else argv)
    if argv and argv[0] in DEVICE_FLAGS:
        argv = argv[1:]
    elif argv and argv[0].startswith("--") and argv[0] in ("--cpu", "--nvidia", "--cambricon", "--ascend",
                                                           "--metax", "--moore", "--iluvatar"):
        print("this engine runs on AMD MI355X only; use --amd")
        print(USAGE)
        sys.exit(1)
    if not argv or argv[0].startswith("--"):
        print(USAGE)
        sys.exit(1)
    model_path = argv.pop(0)
    ndev = 1
    if argv and not argv[0].startswith("--"):
        ndev = int(argv.pop(0))
    import argparse
    ap = argparse.ArgumentParser(usage=USAGE)
    ap.add_argument("--dtype", default="bfloat16", choices=sorted(_DTYPES))
    ap.add_argument("--max-tokens", type=int, default=None)
    ap.add_argument("--prompt", default="山东最高的山是？")
    ap.add_argument("--prompt-ids", default=None)
    ap.add_argument("--max-steps", type=int, default=500)
    ap.add_argument("--temperature", type=float, default=1.0)
    ap.add_argument("--topk", type=int, default=1)
    ap.add_argument("--topp", type=float, default=1.0)
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--page-size", type=int, default=64, choices=(16, 32, 64), help="tokens per cache page")
    ap.add_argument("--cache-tokens", type=int, default=None, help="tokens the page pool holds (default: four contexts)")
    args = ap.parse_args(argv)
    model = MiniCPMForCausalLM(model_path, "cuda:0", ndev, max_tokens=args.max_tokens, dtype=_DTYPES[args.dtype],
                               cache_tokens=args.cache_tokens, page_size=args.page_size)
    prompt = [int(t) for t in args.prompt_ids.split(",")] if args.prompt_ids else args.prompt
    model.generate(prompt, args.max_steps, topp_=args.topp, topk_=args.topk, temperature_=args.temperature,
                   seed=args.seed)
    model.destroy_model_instance()


if __name__ == "__main__":
    test()
