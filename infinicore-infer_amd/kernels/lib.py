"""Loading of the HIP kernel library through ctypes.

The library is searched for under ``lib/`` next to the package (and in the
per-user temporary build folder); when none matches the sources it is built on
the spot.  There is no fallback: without hipcc and without a built library
``get_lib`` raises.
"""
import ctypes
import threading

from . import build as _build


class KernelError(RuntimeError):
    """A kernel entry point refused its arguments or the launch failed."""


_lock = threading.Lock()
_lib = None
_lib_path = None

_c = ctypes
_P = _c.c_void_p
_I = _c.c_int
_F = _c.c_float
_LL = _c.c_longlong



class IcRowFactor(_c.Structure):
    """Row factors rsqrt(sum / width + eps) owed by the rows of an operand (see the C header)."""
    _fields_ = [("sumsq", _P), ("n_parts", _I), ("width", _I), ("eps", _F)]


class IcResidualNorm(_c.Structure):
    """Residual add and norm weight in a product's epilogue (see the C header)."""
    _fields_ = [("x", _P), ("ldx", _I), ("weight", _P), ("alpha", _F), ("sumsq_out", _P), ("n_parts", _I)]


_RF = _c.POINTER(IcRowFactor)
_RN = _c.POINTER(IcResidualNorm)

_SIGNATURES = {
    "ic_embed": [_P, _P, _I, _P, _I, _I, _F, _P],
    "ic_rmsnorm": [_P, _P, _P, _P, _I, _I, _I, _F, _F, _P],
    "ic_add_rmsnorm": [_P, _P, _I, _F, _P, _P, _I, _I, _I, _F, _P],
    "ic_residual_add": [_P, _P, _I, _F, _LL, _P],
    "ic_swiglu": [_P, _P, _I, _I, _I, _P],
    "ic_rope_kv_write": [_P, _I, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _P],
    "ic_attn_generic": [_P, _I, _P, _I, _I, _P, _P, _P, _I, _P, _P, _I, _I, _I, _I, _I, _F, _I, _P],
    "ic_attn_decode_supported": [_I, _I],
    "ic_attn_decode": [_P, _I, _P, _I, _I, _P, _P, _P, _I, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _F, _I, _I, _P],
    "ic_attn_prefill_supported": [_I, _I, _I],
    "ic_attn_prefill_tile_rows": [],
    "ic_attn_prefill": [_P, _I, _P, _I, _I, _P, _P, _P, _I, _P, _I, _I, _I, _I, _I, _F, _I, _P],
    "ic_attn_prefill_groups": [_P, _I, _P, _I, _I, _P, _P, _P, _I, _P, _I, _I, _I, _I, _I, _F, _I, _I, _P],
    "ic_sample": [_P, _LL, _I, _I, _P, _P, _P, _P, _P, _P],
    "ic_argmax": [_P, _LL, _I, _I, _P, _P, _P, _P],
    "ic_argmax_static_max_rows": [],
    "ic_argmax_static": [_P, _LL, _I, _I, _P, _P],
    "ic_gemm_nt": [_P, _I, _P, _I, _P, _I, _I, _I, _I, _I, _I, _I, _F, _I, _RF, _RN, _P],
    "ic_gemm_nt_residual_parts": [_I],
    "ic_gemm_nt_supported": [_I, _I, _I],
    "ic_gemm_qkv_rope_supported": [_I, _I],
    "ic_gemm_qkv_rope": [_P, _P, _P, _I, _I, _I, _I, _I, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _RF, _P],
    "ic_matmul_supported": [_I, _I],
    "ic_matmul": [_P, _I, _P, _P, _I, _I, _I, _I, _I, _I, _I, _F, _P, _LL, _P],
    "ic_matmul_tune": [_P, _I, _P, _P, _I, _I, _I, _I, _I, _I, _I, _P, _LL, _P, _LL, _I, _P],
    "ic_gemm_qkv_rope_tile_rows": [_I],
    "ic_gemm_nt_cfg": [_P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _F, _I, _I, _I, _P],
}


def get_lib():
    global _lib, _lib_path
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is None:
            path = _build.find_library()
            if path is None:
                path = _build.build()
            lib = ctypes.CDLL(path)
            for name, argtypes in _SIGNATURES.items():
                try:
                    fn = getattr(lib, name)
                except AttributeError:
                    raise KernelError("kernel library %s lacks %s" % (path, name))
                fn.argtypes = argtypes
                fn.restype = _I
            _lib, _lib_path = lib, path
    return _lib


def library_path():
    get_lib()
    return _lib_path


def check(status: int, what: str) -> None:
    if status == 0:
        return
    if status == -1:
        raise KernelError("%s: bad argument (shape, stride, alignment or size outside what the kernel takes)" % what)
    if status == -2:
        raise KernelError("%s: unsupported dtype or head size" % what)
    if status == -5:
        raise KernelError("%s: more rows than the entry point's fixed scratch memory holds" % what)
    raise KernelError("%s: HIP error %d at launch" % (what, status))
