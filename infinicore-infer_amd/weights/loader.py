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
vectors (norm weights) are held in float32.  Integer tables become int32.  A
matrix or vector stored as anything but a floating-point type of 16 bits or
more (a quantized checkpoint) is an error that names the tensor.

Upload: all tensors go into one device allocation (the reference copies tensor
by tensor, synchronously, under a global mutex: src/tensor/tensor.cpp:142-167).
Tensors are converted on the host into one of two pinned staging buffers and
copied from there asynchronously; the load synchronises once, at the end.
"""
import fnmatch
import glob
import os
import time
from dataclasses import dataclass
from typing import Dict, Iterable, List, Optional, Tuple

import torch
from safetensors import safe_open


class WeightError(ValueError):
    """The weight files do not match what the model needs."""

    def __init__(self, model_dir, missing, unexpected, wrong_shape, other=(), wrong_dtype=()):
        self.missing = list(missing)
        self.unexpected = list(unexpected)
        self.wrong_shape = list(wrong_shape)
        self.wrong_dtype = list(wrong_dtype)
        self.other = list(other)
        lines = ["weights in %s do not match the model:" % model_dir]
        if self.missing:
            lines.append("  missing tensors (%d): %s" % (len(self.missing), ", ".join(self.missing)))
        if self.unexpected:
            lines.append("  unexpected tensors (%d): %s" % (len(self.unexpected), ", ".join(self.unexpected)))
        if self.wrong_shape:
            lines.append("  wrong shapes (%d): %s" % (len(self.wrong_shape), "; ".join(
                "%s is %s, expected %s" % (n, list(got), list(want)) for n, got, want in self.wrong_shape)))
        if self.wrong_dtype:
            lines.append("  wrong dtypes (%d): %s" % (len(self.wrong_dtype), "; ".join(
                "%s is stored as %s, expected %s" % (n, got, want) for n, got, want in self.wrong_dtype)))
        for o in self.other:
            lines.append("  " + o)
        super().__init__("\n".join(lines))


@dataclass(frozen=True)
class WeightSpec:
    """What a part needs of one tensor.  role: 'matrix' (a GEMM operand or a
    table, keeps its stored dtype), 'vector' (a scale vector, float32) or
    'int' (an integer table, int32).  ``fallback``: another tensor's name that
    stands in when this one is absent from the files (tied embeddings).
    ``tied``: the configuration says this tensor IS its fallback; when the files
    hold both they must be equal, and one copy is kept.  ``pack`` = (name, place):
    tensors with the same pack name are laid out one after the other in the order
    of ``place``, and the loader also hands out their concatenation along the rows
    under that name without copying (fused projections)."""
    shape: Tuple[int, ...]
    role: str = "matrix"
    fallback: Optional[str] = None
    tied: bool = False
    pack: Optional[Tuple[str, int]] = None


# Non-parameter buffers that some exporters write; never needed, never an error.
IGNORED_PATTERNS = ("*.rotary_emb.inv_freq", "*.rotary_emb.cos_cached", "*.rotary_emb.sin_cached")

# safetensors dtype names a role accepts.  Anything else (8-bit floats, integers where a matrix is
# expected: a quantized checkpoint) is refused by tensor name instead of being converted silently.
_FLOAT_NAMES = ("F64", "F32", "BF16", "F16")
_INT_NAMES = ("I64", "I32", "I16", "I8", "U8", "U16", "U32", "U64")
_TORCH_OF = {"F64": torch.float64, "F32": torch.float32, "BF16": torch.bfloat16, "F16": torch.float16}

_ALIGN = 256                # bytes: every tensor of the arena starts on such a boundary
_STAGE_BYTES = 128 << 20    # size of each of the two pinned staging buffers

last_load_report: Dict[str, float] = {}     # seconds and bytes of the most recent load_weights call


def _safetensors_files(model_dir: str) -> List[str]:
    files = sorted(glob.glob(os.path.join(model_dir, "*.safetensors")))
    if not files:
        raise WeightError(model_dir, [], [], [], ["no *.safetensors file in the folder"])
    return files


def _target_dtype(stored: torch.dtype, role: str, compute_dtype: torch.dtype) -> torch.dtype:
    if role == "int":
        return torch.int32
    if role == "vector" or compute_dtype == torch.float32:
        return torch.float32
    if stored in (torch.float32, torch.bfloat16):
        return stored
    return compute_dtype


def _nbytes(shape, dtype) -> int:
    n = 1
    for s in shape:
        n *= int(s)
    return n * torch.empty((), dtype=dtype).element_size()


class _Uploader:
    """Copies host tensors into slices of one device arena through two pinned staging buffers,
    asynchronously: while one buffer's copy to the device runs, the next tensor is converted into the
    other.  One synchronisation at the end.  On a CPU 'device' the slices are written directly."""

    def __init__(self, arena: torch.Tensor):
        self.arena = arena
        self.cuda = arena.is_cuda
        if self.cuda:
            self.stage = [torch.empty(_STAGE_BYTES, dtype=torch.uint8, pin_memory=True) for _ in range(2)]
            self.events = [None, None]
            self.turn = 0
            self.stream = torch.cuda.Stream(device=arena.device)

    def put(self, offset: int, src: torch.Tensor, dtype: torch.dtype) -> None:
        """arena[offset ...] = src converted to dtype (src on the host, any float or integer dtype)."""
        src = src.reshape(-1)
        item = torch.empty((), dtype=dtype).element_size()
        total = src.numel()
        if not self.cuda:
            self.arena[offset:offset + total * item].view(dtype).copy_(src)
            return
        per = _STAGE_BYTES // item
        for lo in range(0, total, per):
            n = min(per, total - lo)
            i = self.turn
            self.turn ^= 1
            if self.events[i] is not None:
                self.events[i].synchronize()            # the last copy out of this buffer is done
            host = self.stage[i][:n * item].view(dtype)
            host.copy_(src[lo:lo + n])                   # the dtype conversion happens here, on the host
            with torch.cuda.stream(self.stream):
                self.arena[offset + lo * item:offset + (lo + n) * item].copy_(self.stage[i][:n * item],
                                                                              non_blocking=True)
                ev = self.events[i] or torch.cuda.Event()
                ev.record(self.stream)
                self.events[i] = ev

    def finish(self) -> None:
        if self.cuda:
            self.stream.synchronize()
            torch.cuda.current_stream(self.arena.device).wait_stream(self.stream)


def load_weights(model_dir: str, specs: Dict[str, WeightSpec], compute_dtype: torch.dtype,
                 device="cpu", ignored: Iterable[str] = IGNORED_PATTERNS) -> Dict[str, torch.Tensor]:
    """Load the tensors named by ``specs`` into ONE allocation on ``device`` (an arena; every tensor
    handed out is a view of it) and return them by name, plus one entry per pack name.  A spec whose
    tensor is absent but whose fallback is present gets the fallback's tensor (the SAME tensor object
    when both names are wanted: a tied table is held once).  Everything that is wrong with the files
    is reported in one ``WeightError``."""
    t_start = time.time()
    files = _safetensors_files(model_dir)
    where: Dict[str, str] = {}
    shapes: Dict[str, Tuple[int, ...]] = {}
    stored: Dict[str, str] = {}
    for path in files:
        with safe_open(path, "pt") as f:
            for name in f.keys():
                sl = f.get_slice(name)
                where[name] = path
                shapes[name] = tuple(sl.get_shape())
                stored[name] = str(sl.get_dtype())

    resolved: Dict[str, str] = {}
    missing, wrong, wrong_dtype = [], [], []
    tied_pairs = []
    for name, spec in specs.items():
        src = name if name in where else (spec.fallback if spec.fallback in where else None)
        if src is None:
            missing.append(name if not spec.fallback else "%s (or %s)" % (name, spec.fallback))
            continue
        if spec.tied and name in where and spec.fallback in where:
            tied_pairs.append((name, spec.fallback))
        resolved[name] = src
        if tuple(shapes[src]) != tuple(spec.shape):
            wrong.append((src, shapes[src], spec.shape))
        ok = _INT_NAMES if spec.role == "int" else _FLOAT_NAMES
        if stored[src] not in ok and not any(src == w[0] for w in wrong_dtype):
            wrong_dtype.append((src, stored[src], "an integer type" if spec.role == "int"
                                else "a floating-point type (%s)" % ", ".join(_FLOAT_NAMES)))
    used = set(resolved.values())
    unexpected = sorted(n for n in where if n not in used
                        and not any(fnmatch.fnmatch(n, p) for p in ignored))
    if missing or wrong or unexpected or wrong_dtype:
        raise WeightError(model_dir, sorted(missing), unexpected, wrong, wrong_dtype=wrong_dtype)

    # ---- tensors the configuration calls tied although the files hold both ----------------------
    other = []
    for name, fb in tied_pairs:
        with safe_open(where[name], "pt") as f:
            a = f.get_tensor(name)
        with safe_open(where[fb], "pt") as f:
            b = f.get_tensor(fb)
        if a.dtype == b.dtype and torch.equal(a, b):
            resolved[name] = resolved.get(fb, fb)          # equal: one copy serves both names
        else:
            other.append("%s and %s are both present and differ although the configuration ties them"
                         % (name, fb))
    if other:
        raise WeightError(model_dir, [], [], [], other)

    # ---- the arena's layout: one place per (source tensor, target dtype); packs are contiguous ---
    device = torch.device(device)
    target: Dict[str, torch.dtype] = {}
    for name, src in resolved.items():
        st = _TORCH_OF.get(stored[src], torch.int64)
        target[name] = _target_dtype(st, specs[name].role, compute_dtype)
    packs: Dict[str, List[Tuple[int, str]]] = {}
    for name, spec in specs.items():
        if spec.pack is not None and name in resolved:
            packs.setdefault(spec.pack[0], []).append((spec.pack[1], name))
    place: Dict[Tuple[str, torch.dtype], int] = {}
    packed_ok: Dict[str, Tuple[int, torch.dtype, Tuple[int, ...]]] = {}
    total = 0

    def reserve(key, nbytes, align=True):
        nonlocal total
        if align:
            total = (total + _ALIGN - 1) // _ALIGN * _ALIGN
        place[key] = total
        total += nbytes

    for pname, members in packs.items():
        members.sort()
        names = [n for _, n in members]
        dts = {target[n] for n in names}
        inner = {tuple(specs[n].shape[1:]) for n in names}
        keys = [(resolved[n], target[n]) for n in names]
        if len(dts) == 1 and len(inner) == 1 and not any(k in place for k in keys) and len(set(keys)) == len(keys):
            dt = dts.pop()
            first = True
            for n, k in zip(names, keys):
                reserve(k, _nbytes(specs[n].shape, dt), align=first)
                first = False
            rows = sum(specs[n].shape[0] for n in names)
            packed_ok[pname] = (place[keys[0]], dt, (rows,) + tuple(specs[names[0]].shape[1:]))
    for name, src in resolved.items():
        key = (src, target[name])
        if key not in place:
            reserve(key, _nbytes(specs[name].shape, target[name]))

    arena = torch.empty(max(total, 1), dtype=torch.uint8, device=device)
    up = _Uploader(arena)
    by_file: Dict[str, List[Tuple[str, torch.dtype]]] = {}
    for key in place:
        by_file.setdefault(where[key[0]], []).append(key)
    for path, keys in by_file.items():
        with safe_open(path, "pt") as f:
            for src, dt in sorted(keys, key=lambda k: place[k]):
                up.put(place[(src, dt)], f.get_tensor(src), dt)
    up.finish()

    out: Dict[str, torch.Tensor] = {}
    views: Dict[Tuple[str, torch.dtype], torch.Tensor] = {}
    for name, src in resolved.items():
        dt = target[name]
        key = (src, dt)
        if key not in views:                 # two names of one stored tensor get the same tensor object
            o = place[key]
            views[key] = arena[o:o + _nbytes(specs[name].shape, dt)].view(dt).view(*specs[name].shape)
        out[name] = views[key]
    for pname, (o, dt, shape) in packed_ok.items():
        out[pname] = arena[o:o + _nbytes(shape, dt)].view(dt).view(*shape)
    last_load_report.clear()
    last_load_report.update(seconds=time.time() - t_start, bytes=float(total), tensors=float(len(place)),
                            files=float(len(files)))
    return out
