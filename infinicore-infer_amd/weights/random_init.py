"""Random-weights mode: a model folder (config.json, model.safetensors) from a
configuration and a seed.  The reference has no such mode; its tensor names
and shapes (scripts/jiuge.py:33-77) are what the folder holds.

A value is a function of (seed, tensor name, element index) alone: it depends
neither on the order in which tensors are drawn, nor on the device that draws
them, nor on how a tensor is cut into pieces while it is drawn.  So a folder
written on the CPU and weights drawn straight into a model on the GPU are the
same model.  Matrices and tables are N(0, std) in float32, rounded to the storage
dtype; norm weights are 1, or N(1, norm_std).

The draw uses integer arithmetic and one multiplication only, which give the same
bits everywhere: two 64-bit words per element from a counter hash (splitmix64's
finaliser over key + index * odd constant), cut into eight 16-bit uniforms whose
sum, centred and scaled, is close to a standard normal (Irwin-Hall with n = 8:
variance exact, tails end at 4.9 sigma).
"""
import hashlib
import json
import os
from typing import Dict, Optional

import torch
from safetensors.torch import save_file

from ..config.registry import config_from_dict

_M64 = (1 << 64) - 1
_GOLDEN = 0x9E3779B97F4A7C15
_MIX1 = 0xBF58476D1CE4E5B9
_MIX2 = 0x94D049BB133111EB
_CHUNK = 1 << 24                                        # elements drawn at a time on a GPU (bounds the temporaries)
_CHUNK_CPU = 1 << 18                                    # on the CPU: pieces that stay in its caches (20 times faster)


def _key(seed: int, name: str) -> int:
    h = hashlib.sha256(("%d:%s" % (seed, name)).encode()).digest()
    return int.from_bytes(h[:8], "little")


def _i64(v: int) -> int:
    """The int64 with the bit pattern of the unsigned 64-bit v."""
    v &= _M64
    return v - (1 << 64) if v >= (1 << 63) else v


def _shr(x: torch.Tensor, s: int) -> torch.Tensor:
    """Logical shift right of int64 bit patterns."""
    return (x >> s) & ((1 << (64 - s)) - 1)


def _mixed(x: torch.Tensor) -> torch.Tensor:
    x = x ^ _shr(x, 30)
    x = x * _i64(_MIX1)
    x = x ^ _shr(x, 27)
    x = x * _i64(_MIX2)
    return x ^ _shr(x, 31)


def standard_normal(seed: int, name: str, n: int, device="cpu") -> torch.Tensor:
    """n float32 values, element i a function of (seed, name, i) only."""
    key = _key(seed, name)
    out = torch.empty(n, dtype=torch.float32, device=device)
    scale = (1.5 ** 0.5) / 65536.0
    chunk = _CHUNK_CPU if torch.device(device).type == "cpu" else _CHUNK
    for start in range(0, n, chunk):
        stop = min(n, start + chunk)
        i = torch.arange(start, stop, dtype=torch.int64, device=device)
        total = torch.zeros(stop - start, dtype=torch.int64, device=device)
        for word in (0, 1):
            x = _mixed(i * _i64(_GOLDEN) + _i64(key + word * _MIX2))
            for field in range(4):
                total += (x >> (16 * field)) & 0xFFFF
        # sum of eight uniforms (field + 1/2) / 65536, minus its mean 4, times sqrt(12 / 8): one exact float64 product
        out[start:stop] = ((total - (4 * 65536 - 4)).to(torch.float64) * scale).to(torch.float32)
    return out


def _draw(seed: int, name: str, shape, role: str, std: float, norm_std: float, device) -> torch.Tensor:
    n = 1
    for d in shape:
        n *= int(d)
    if role == "vector":
        t = torch.ones(shape, dtype=torch.float32, device=device)
        if norm_std:
            t = t + norm_std * standard_normal(seed, name, n, device).view(shape)
        return t
    if role == "int":
        raise ValueError("no rule to draw integer tensor %s" % name)
    return std * standard_normal(seed, name, n, device).view(shape)


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
    specs = model.weight_specs()
    for name, spec in specs.items():
        if tie and spec.fallback in specs and spec.fallback in out:
            continue                # a tied tensor is not written: the loader takes the tensor it falls back to
        t = _draw(seed, name, spec.shape, spec.role, std, norm_std, device)
        out[name] = (t if spec.role == "vector" else t.to(dtype)).contiguous()
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
        t = _draw(seed, name, spec.shape, spec.role, std, norm_std, rt.device)
        tensors[name] = t if spec.role == "vector" else t.to(rt.dtype)
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
