"""Random-weights mode: a model folder (config.json, model.safetensors) from a
configuration and a seed.  The reference has no such mode; its tensor names
and shapes (scripts/jiuge.py:33-77) are what the folder holds.

Every tensor gets its own generator seeded from (seed, tensor name), so a
value does not depend on the order in which tensors are drawn.  Matrices and
tables are N(0, std) in float32, rounded to the storage dtype; norm weights
are 1, or N(1, norm_std).
"""
import hashlib
import json
import os
from typing import Dict, Optional

import torch
from safetensors.torch import save_file

from ..config.registry import config_from_dict


def _generator(seed: int, name: str, device="cpu") -> torch.Generator:
    h = hashlib.sha256(("%d:%s" % (seed, name)).encode()).digest()
    g = torch.Generator(device=device)
    g.manual_seed(int.from_bytes(h[:8], "little") & 0x7FFFFFFFFFFFFFFF)
    return g


def random_state_dict(config: dict, seed: int, std: float = 0.02, norm_std: float = 0.0,
                      dtype: torch.dtype = torch.bfloat16, device="cpu",
                      tie: Optional[bool] = None) -> Dict[str, torch.Tensor]:
    """Tensors by checkpoint name for ``config`` (a config.json dictionary)."""
    from ..parts import Runtime, build_model          # late: parts import the kernels package
    cfg = config_from_dict(config)
    model = build_model(cfg.model_spec(), Runtime(dtype=dtype, device="cpu"))
    if tie is None:
        tie = config.get("tie_word_embeddings", True)
    out: Dict[str, torch.Tensor] = {}
    for name, spec in model.weight_specs().items():
        if tie and name == "lm_head.weight":
            continue
        g = _generator(seed, name, device)
        if spec.role == "vector":
            t = torch.ones(spec.shape, dtype=torch.float32, device=device)
            if norm_std:
                t = t + norm_std * torch.randn(spec.shape, generator=g, dtype=torch.float32, device=device)
        elif spec.role == "int":
            raise ValueError("no rule to draw integer tensor %s" % name)
        else:
            t = std * torch.randn(spec.shape, generator=g, dtype=torch.float32, device=device)
        out[name] = t.to(dtype).contiguous()
    return out


def init_random_weights(model, seed: int, std: float = 0.02, norm_std: float = 0.0, tie: bool = True) -> None:
    """Random weights straight into a built model, drawn on the model's device
    (no folder is written).  Same rules as ``random_state_dict``; matrices are
    rounded to the model's compute dtype, norm weights stay float32."""
    rt = model.runtime
    specs = model.weight_specs()
    tensors: Dict[str, torch.Tensor] = {}
    for name, spec in specs.items():
        if tie and spec.fallback in specs and spec.fallback in tensors:
            tensors[name] = tensors[spec.fallback]
            continue
        g = _generator(seed, name, rt.device)
        if spec.role == "vector":
            t = torch.ones(spec.shape, dtype=torch.float32, device=rt.device)
            if norm_std:
                t = t + norm_std * torch.randn(spec.shape, generator=g, dtype=torch.float32, device=rt.device)
        else:
            t = (std * torch.randn(spec.shape, generator=g, dtype=torch.float32, device=rt.device)).to(rt.dtype)
        tensors[name] = t
    model.load_weights(tensors)


def write_random_model(folder: str, config: dict, seed: int, std: float = 0.02, norm_std: float = 0.0,
                       dtype: torch.dtype = torch.bfloat16) -> str:
    """Write config.json and model.safetensors into ``folder``; returns it."""
    os.makedirs(folder, exist_ok=True)
    sd = random_state_dict(config, seed, std, norm_std, dtype)
    cfg = dict(config)
    cfg.setdefault("torch_dtype", {torch.bfloat16: "bfloat16", torch.float32: "float32",
                                   torch.float16: "float16"}[dtype])
    with open(os.path.join(folder, "config.json"), "w", encoding="utf-8") as f:
        json.dump(cfg, f, indent=1)
    save_file(sd, os.path.join(folder, "model.safetensors"), metadata={"format": "pt", "seed": str(seed)})
    return folder


def main(argv=None) -> int:
    """python -m infinicore_infer_amd.weights --config config.json --seed S --out DIR
    writes a model folder (config.json, model.safetensors) with random weights for that configuration."""
    import argparse
    ap = argparse.ArgumentParser(prog="python -m infinicore_infer_amd.weights", description="write a model folder with random weights")
    ap.add_argument("--config", required=True, help="a config.json of the architecture")
    ap.add_argument("--out", required=True, help="folder to write (created if missing)")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--std", type=float, default=0.02, help="standard deviation of matrices and embeddings")
    ap.add_argument("--norm-std", type=float, default=0.0, help="norm weights are 1 + N(0, this)")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    args = ap.parse_args(argv)
    with open(args.config, encoding="utf-8") as f:
        config = json.load(f)
    folder = write_random_model(args.out, config, args.seed, args.std, args.norm_std,
                                {"bfloat16": torch.bfloat16, "float32": torch.float32}[args.dtype])
    print("wrote %s" % folder)
    return 0
