"""y = x W^T for weights stored [out, in] (the checkpoint's layout; the
reference views them transposed, src/models/jiuge/jiuge_weight.hpp:51-54).

The matrix product itself is a library routine for many rows, as in the
reference (inference_context.cpp:59-79 calls the library's Gemm), and the
package's own matrix-core kernel for few rows (decoding, the output head).
float32 operands always go to the library with reduced-precision matrix modes
switched off.
"""
import torch

from ..kernels import ops
from .base import DeferredRows

# float32 products must be true float32.
torch.backends.cuda.matmul.allow_tf32 = False
torch.backends.cudnn.allow_tf32 = False

# Which product runs where (own kernel up to some rows, slices over K for the projections into the residual
# stream, the library beyond) is the kernel library's rule, asked through ops.rule_*: its native step function
# asks the same functions, so the two ways of issuing a step choose alike.
TUNE_LIBRARY = False   # while True, every library product times the library's algorithms for its shape first
TUNE_FLUSH = None      # while tuning: a tensor larger than the caches, overwritten before every timed launch
_tuned = set()


def _library(x, w, out, alpha: float = 1.0):
    """out = alpha * x w^T through the library, as the reference does for every product
    (inference_context.cpp:59-79): hipBLASLt called directly, torch's routine if it has no
    algorithm for the shape."""
    if TUNE_LIBRARY:
        key = (x.dtype, out.dtype, x.shape[0], w.shape[0], w.shape[1], x.stride(0), w.stride(0), out.stride(0))
        if key not in _tuned:
            _tuned.add(key)
            try:
                ops.matmul_library_tune(x, w, out, flush=TUNE_FLUSH)
            except ops.KernelError:
                pass
    try:
        return ops.matmul_library(x, w, out, alpha)
    except ops.NoLibraryAlgorithm:
        if out.dtype == x.dtype:
            torch.mm(x, w.t(), out=out)
        else:
            out.copy_(torch.mm(x.to(out.dtype), w.to(out.dtype).t()))
        return out.mul_(alpha) if alpha != 1.0 else out


def own_kernel_applies(M, x_dtype, w_dtype, out_dtype, impl: str) -> bool:
    return impl == "auto" and ops.rule_own_product(x_dtype, w_dtype, out_dtype, M)


def linear(x, w, out, impl: str = "auto", alpha: float = 1.0, ws=None):
    """out[M, N] = alpha * x[M, K] @ w[N, K]^T.  out may be float32 when x is bfloat16.  x may be
    ``DeferredRows``: the row factors are applied to the result by the own kernel, or to x first.
    ``ws``: the step's workspace, for the float32 copies that a matrix stored in 32-bit under a bfloat16
    model needs (without it they are allocated by the call)."""
    if isinstance(x, DeferredRows):
        if own_kernel_applies(x.shape[0], x.dtype, w.dtype, out.dtype, impl):
            return ops.gemm_nt(x.values, w, out, alpha=alpha, row_factor=x.row_factor())
        x = x.materialize()
    if w.dtype != x.dtype:
        # a matrix stored in 32-bit stays so: compute this product in float32
        # (w is the 32-bit one, so only the few activations are converted; no copy of the matrix is made)
        def scratch(name, shape):
            if ws is None:
                return torch.empty(shape, dtype=torch.float32, device=out.device)
            return ws.buffer(name, shape, torch.float32)
        x32 = x if x.dtype == torch.float32 else scratch("linear_x32", tuple(x.shape)).copy_(x)
        w32 = w if w.dtype == torch.float32 else w.to(torch.float32)
        if out.dtype == torch.float32:
            return _library(x32, w32, out, alpha)
        tmp = scratch("linear_out32", tuple(out.shape))
        _library(x32, w32, tmp, alpha)
        out.copy_(tmp)
        return out
    if own_kernel_applies(x.shape[0], x.dtype, w.dtype, out.dtype, impl):
        return ops.gemm_nt(x, w, out, alpha=alpha)
    return _library(x, w, out, alpha)


def linear_tail(x, w, tail, ws, name: str, impl: str = "auto"):
    """The last projection of a part with the residual add and the following norm's weight in its
    epilogue: returns ``DeferredRows`` for that norm, or None when this step cannot be done so
    (many rows, float32, a width beyond the kernel's) and the caller computes the plain product."""
    M, N = x.shape[0], w.shape[0]
    if tail is None or impl != "auto" or tuple(tail.x.shape) != (M, N) or x.stride(1) != 1 or w.stride(1) != 1:
        return None
    how = ops.rule_tail(x.dtype, x, w)
    if how == ops.TAIL_PLAIN:
        return None
    if how == ops.TAIL_SLICES:
        # 17..64 rows into the residual stream (and 13..16 long ones): the product as slices over K; the kernel that
        # sums them does the add and the whole norm, so the rows handed on owe nothing
        slices = ops.gemm_splitk_slices(N, w.shape[1])
        parts = ops.gemm_splitk(x, w, ws.buffer("tail_parts", (slices * M * N,), torch.float32), slices)
        y = ws.buffer(name + "_values", (M, N), torch.bfloat16)
        ops.splitk_add_rmsnorm(parts, tail.x, tail.alpha, tail.weight, y, tail.eps)
        return DeferredRows(y, None, N, tail.eps)
    parts = ops.residual_parts(N)
    y = ws.buffer(name + "_values", (M, N), torch.bfloat16)
    sumsq = ws.buffer(name + "_sumsq", (parts, 16), torch.float32)
    ops.gemm_nt(x, w, y, residual=(tail.x, tail.weight, tail.alpha, sumsq))
    return DeferredRows(y, sumsq, N, tail.eps)
