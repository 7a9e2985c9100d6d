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

# float32 products must be true float32.
torch.backends.cuda.matmul.allow_tf32 = False
torch.backends.cudnn.allow_tf32 = False

FEW_ROWS = 16          # up to here the package's own kernel beats the library on MI355X
_mm_out_dtype_ok = None


def _library_mm_f32_out(x, w, out):
    """bfloat16 operands, float32 result: the library's mixed-output product when it has one."""
    global _mm_out_dtype_ok
    if _mm_out_dtype_ok is None:
        try:
            torch.mm(x[:1], w[:1].t(), out_dtype=torch.float32)
            _mm_out_dtype_ok = True
        except Exception:
            _mm_out_dtype_ok = False
    if _mm_out_dtype_ok:
        try:
            torch.mm(x, w.t(), out_dtype=torch.float32, out=out)
        except (TypeError, RuntimeError):
            out.copy_(torch.mm(x, w.t(), out_dtype=torch.float32))
    else:
        ops.gemm_nt(x, w, out)


def own_kernel_applies(M, x_dtype, w_dtype, out_dtype, impl: str) -> bool:
    return (impl == "auto" and M <= FEW_ROWS and x_dtype == torch.bfloat16 and w_dtype == torch.bfloat16
            and ops.gemm_nt_supported(x_dtype, w_dtype, out_dtype))


def linear(x, w, out, impl: str = "auto", alpha: float = 1.0):
    """out[M, N] = alpha * x[M, K] @ w[N, K]^T.  out may be float32 when x is bfloat16.  x may be
    ``DeferredRows``: the row factors are applied to the result by the own kernel, or to x first."""
    from .base import DeferredRows
    if isinstance(x, DeferredRows):
        if own_kernel_applies(x.shape[0], x.dtype, w.dtype, out.dtype, impl):
            return ops.gemm_nt(x.values, w, out, alpha=alpha, row_factor=x.row_factor())
        x = x.materialize()
    if alpha != 1.0:
        if own_kernel_applies(x.shape[0], x.dtype, w.dtype, out.dtype, impl):
            return ops.gemm_nt(x, w, out, alpha=alpha)
        linear(x, w, out, impl)
        return out.mul_(alpha)
    if w.dtype != x.dtype:
        # a matrix stored in 32-bit stays so: compute this product in float32
        tmp = torch.mm(x.to(torch.float32), w.to(torch.float32).t())
        out.copy_(tmp)
        return out
    M = x.shape[0]
    if x.dtype == torch.bfloat16:
        if (impl == "auto" and M <= FEW_ROWS) and ops.gemm_nt_supported(x.dtype, w.dtype, out.dtype):
            return ops.gemm_nt(x, w, out)
        if out.dtype == torch.float32:
            _library_mm_f32_out(x, w, out)
            return out
    torch.mm(x, w.t(), out=out)
    return out


def linear_tail(x, w, tail, ws, name: str, impl: str = "auto"):
    """The last projection of a part with the residual add and the following norm's weight in its
    epilogue: returns ``DeferredRows`` for that norm, or None when this step cannot be done so
    (many rows, float32, a width beyond the kernel's) and the caller computes the plain product."""
    from .base import DeferredRows
    M, N = x.shape[0], w.shape[0]
    if tail is None or not own_kernel_applies(M, x.dtype, w.dtype, torch.bfloat16, impl):
        return None
    parts = ops.residual_parts(N)
    if parts > ops.MAX_SUMSQ_PARTS or tuple(tail.x.shape) != (M, N):
        return None
    y = ws.buffer(name + "_values", (M, N), torch.bfloat16)
    sumsq = ws.buffer(name + "_sumsq", (parts, 16), torch.float32)
    ops.gemm_nt(x, w, y, residual=(tail.x, tail.weight, tail.alpha, sumsq))
    return DeferredRows(y, sumsq, N, tail.eps)
