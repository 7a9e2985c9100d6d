"""Weights from safetensors, looked up by tensor name.

The reference reads every ``*.safetensors`` file of the folder in sorted order
into one dictionary (scripts/jiuge.py:400-407) and then indexes it by the
checkpoint's names (scripts/jiuge.py:33-77).  Here the model's parts say which
names, shapes and roles they need (``WeightSpec``); the loader compares that
with what the files hold and raises ONE error that lists every missing tensor,
every unexpected tensor and every wrong shape.

Storage rule: matrices and tables stay in the dtype they are stored in when
that is bfloat16 or float32 (float16 is converted to the compute dtype); with
compute dtype float32 everything becomes float32.  One-dimensional scale
vectors (norm weights) are held in float32.  Integer tensors become int32.
"""
import fnmatch
import glob
import os
from dataclasses import dataclass
from typing import Dict, Iterable, List, Optional, Tuple

import torch
from safetensors import safe_open


class WeightError(ValueError):
    """The weight files do not match what the model needs."""

    def __init__(self, model_dir, missing, unexpected, wrong_shape, other=()):
        self.missing = list(missing)
        self.unexpected = list(unexpected)
        self.wrong_shape = list(wrong_shape)
        self.other = list(other)
        lines = ["weights in %s do not match the model:" % model_dir]
        if self.missing:
            lines.append("  missing tensors (%d): %s" % (len(self.missing), ", ".join(self.missing)))
        if self.unexpected:
            lines.append("  unexpected tensors (%d): %s" % (len(self.unexpected), ", ".join(self.unexpected)))
        if self.wrong_shape:
            lines.append("  wrong shapes (%d): %s" % (len(self.wrong_shape), "; ".join(
                "%s is %s, expected %s" % (n, list(got), list(want)) for n, got, want in self.wrong_shape)))
        for o in self.other:
            lines.append("  " + o)
        super().__init__("\n".join(lines))


@dataclass(frozen=True)
class WeightSpec:
    """What a part needs of one tensor.  role: 'matrix' (a GEMM operand or a
    table, keeps its stored dtype), 'vector' (a scale vector, float32) or
    'int' (an integer table, int32).  ``fallback``: another tensor's name that
    stands in when this one is absent from the files (tied embeddings)."""
    shape: Tuple[int, ...]
    role: str = "matrix"
    fallback: Optional[str] = None


# Non-parameter buffers that some exporters write; never needed, never an error.
IGNORED_PATTERNS = ("*.rotary_emb.inv_freq", "*.rotary_emb.cos_cached", "*.rotary_emb.sin_cached")


def _safetensors_files(model_dir: str) -> List[str]:
    files = sorted(glob.glob(os.path.join(model_dir, "*.safetensors")))
    if not files:
        raise WeightError(model_dir, [], [], [], ["no *.safetensors file in the folder"])
    return files


def _target_dtype(stored: torch.dtype, role: str, compute_dtype: torch.dtype) -> torch.dtype:
    if role == "int" or not stored.is_floating_point:
        return torch.int32
    if role == "vector" or compute_dtype == torch.float32:
        return torch.float32
    if stored in (torch.float32, torch.bfloat16):
        return stored
    return compute_dtype


def load_weights(model_dir: str, specs: Dict[str, WeightSpec], compute_dtype: torch.dtype,
                 device="cpu", ignored: Iterable[str] = IGNORED_PATTERNS) -> Dict[str, torch.Tensor]:
    """Load the tensors named by ``specs``.  A spec whose tensor is absent but
    whose fallback is present gets the fallback's tensor (the SAME tensor
    object when both names are wanted: a tied table is held once)."""
    files = _safetensors_files(model_dir)
    where: Dict[str, str] = {}
    shapes: Dict[str, Tuple[int, ...]] = {}
    for path in files:
        with safe_open(path, "pt") as f:
            for name in f.keys():
                where[name] = path
                shapes[name] = tuple(f.get_slice(name).get_shape())

    resolved: Dict[str, str] = {}
    missing, wrong = [], []
    for name, spec in specs.items():
        src = name if name in where else (spec.fallback if spec.fallback in where else None)
        if src is None:
            missing.append(name if not spec.fallback else "%s (or %s)" % (name, spec.fallback))
            continue
        resolved[name] = src
        if tuple(shapes[src]) != tuple(spec.shape):
            wrong.append((src, shapes[src], spec.shape))
    used = set(resolved.values())
    unexpected = sorted(n for n in where if n not in used
                        and not any(fnmatch.fnmatch(n, p) for p in ignored))
    if missing or wrong or unexpected:
        raise WeightError(model_dir, sorted(missing), unexpected, wrong)

    loaded: Dict[Tuple[str, torch.dtype], torch.Tensor] = {}
    out: Dict[str, torch.Tensor] = {}
    by_file: Dict[str, List[str]] = {}
    for name, src in resolved.items():
        by_file.setdefault(where[src], []).append(name)
    for path, names in by_file.items():
        with safe_open(path, "pt") as f:
            for name in names:
                src = resolved[name]
                t = f.get_tensor(src)
                dt = _target_dtype(t.dtype, specs[name].role, compute_dtype)
                key = (src, dt)
                if key not in loaded:
                    loaded[key] = t.to(dtype=dt).to(device).contiguous()
                out[name] = loaded[key]
    return out
