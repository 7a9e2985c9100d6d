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


# ---- the native step function (see csrc/infinicore_infer_engine.h) -----------------------------------
MAX_CACHE_GROUPS = 8


class IcNorm(_c.Structure):
    _fields_ = [("weight", _P), ("eps", _F)]


class IcAttention(_c.Structure):
    _fields_ = [("n_heads", _I), ("n_kv_heads", _I), ("head_dim", _I), ("window", _I), ("shared_kv", _I),
                ("rot_dim", _I), ("max_positions", _I), ("softmax_scale", _F), ("cos", _P), ("sin", _P),
                ("w_qkv", _P), ("w_o", _P)]


class IcSwiGLU(_c.Structure):
    _fields_ = [("intermediate", _I), ("w_gate_up", _P), ("w_down", _P)]


class IcLayer(_c.Structure):
    _fields_ = [("mixer_norm", IcNorm), ("attention", IcAttention), ("ffn_norm", IcNorm), ("ffn", IcSwiGLU),
                ("residual_scale", _F)]


class IcRunEntry(_c.Structure):
    _fields_ = [("layer", _I), ("writes_cache", _I), ("group", _I), ("k_cache", _P), ("v_cache", _P)]


class IcDecoderMeta(_c.Structure):
    _fields_ = [("dtype", _I), ("hidden", _I), ("vocab", _I), ("page_size", _I), ("n_layers", _I), ("n_entries", _I),
                ("n_groups", _I), ("compute_units", _I), ("embed_scale", _F), ("logit_scale", _F),
                ("embed_table", _P), ("head_weight", _P), ("final_norm", IcNorm), ("final_norm_scaled", _P),
                ("attention_counters", _P)]


class IcStepBatch(_c.Structure):
    _fields_ = [("n_tokens", _I), ("n_requests", _I), ("n_want", _I), ("n_decode_rows", _I), ("n_prefill_tiles", _I),
                ("want_rows_identity", _I), ("decode_rows_identity", _I), ("max_position", _I), ("max_context", _I),
                ("fixed_decode_splits", _I), ("tokens", _P), ("positions", _P), ("token_req", _P), ("want_rows", _P),
                ("decode_rows", _P), ("prefill_tiles", _P), ("group_slots", _P * MAX_CACHE_GROUPS),
                ("group_tables", _P * MAX_CACHE_GROUPS), ("group_table_stride", _I * MAX_CACHE_GROUPS)]


class IcHostBatch(_c.Structure):
    _fields_ = [("n_tokens", _I), ("n_requests", _I), ("tokens", _P), ("req_lens", _P), ("req_pos", _P),
                ("want_count", _P), ("want", _P), ("tables", _P), ("table_len", _P), ("tile_rows", _I),
                ("fixed_decode_splits", _I)]


_RF = _c.POINTER(IcRowFactor)
_RN = _c.POINTER(IcResidualNorm)

_SIGNATURES = {
    "ic_embed": [_P, _P, _I, _P, _I, _I, _F, _P],
    "ic_rmsnorm": [_P, _P, _P, _P, _I, _I, _I, _F, _F, _P],
    "ic_add_rmsnorm": [_P, _P, _I, _F, _P, _P, _I, _I, _I, _F, _P],
    "ic_residual_add": [_P, _P, _I, _F, _LL, _P],
    "ic_swiglu": [_P, _P, _I, _I, _I, _P],
    "ic_copy_pages": [_P, _I, _LL, _LL, _P, _P, _I, _P],
    "ic_rope_kv_write": [_P, _I, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _P],
    "ic_attn_generic": [_P, _I, _P, _I, _I, _P, _P, _P, _I, _P, _P, _I, _I, _I, _I, _I, _F, _I, _P],
    "ic_attn_decode_supported": [_I, _I],
    "ic_attn_decode": [_P, _I, _P, _I, _I, _P, _P, _P, _I, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _F, _I, _I, _P],
    "ic_attn_prefill_supported": [_I, _I, _I],
    "ic_attn_prefill_tile_rows": [],
    "ic_attn_prefill": [_P, _I, _P, _I, _I, _P, _P, _P, _I, _P, _I, _I, _I, _I, _I, _F, _I, _P],
    "ic_attn_prefill_groups": [_P, _I, _P, _I, _I, _P, _P, _P, _I, _P, _I, _I, _I, _I, _I, _F, _I, _I, _P],
    "ic_attn_prefill_scratch_floats": [_I, _I, _I, _I],
    "ic_attn_prefill_parts": [_I, _I, _I, _I, _I, _c.POINTER(_I)],
    "ic_attn_prefill_parts_of_step": [_I, _I, _I, _I, _I, _I, _I, _c.POINTER(_I)],
    "ic_attn_prefill_split": [_P, _I, _P, _I, _I, _P, _P, _P, _I, _P, _I, _I, _I, _I, _I, _F, _I, _I, _I, _I, _P, _LL, _P, _P],
    "ic_attn_prefill_counter_ints": [],
    "ic_sample": [_P, _LL, _I, _I, _P, _P, _P, _P, _P, _P],
    "ic_argmax": [_P, _LL, _I, _I, _P, _P, _P, _P],
    "ic_argmax_static_max_rows": [],
    "ic_argmax_static": [_P, _LL, _I, _I, _P, _P],
    "ic_gemm_nt": [_P, _I, _P, _I, _P, _I, _I, _I, _I, _I, _I, _I, _F, _I, _RF, _RN, _P],
    "ic_gemm_nt_residual_parts": [_I],
    "ic_gemm_nt_variant": [_P, _I, _P, _I, _P, _I, _I, _I, _I, _I, _I, _I, _F, _I, _RF, _RN, _I, _P],
    "ic_gemm_nt_epilogue_rows": [_I, _I, _I, _I],
    "ic_peak_mfma_bf16": [_P, _I, _I, _P],
    "ic_peak_read": [_P, _LL, _I, _P, _P],
    "ic_gemm_nt_supported": [_I, _I, _I],
    "ic_gemm_qkv_rope_supported": [_I, _I],
    "ic_gemm_qkv_rope": [_P, _P, _P, _I, _I, _I, _I, _I, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _RF, _P],
    "ic_matmul_supported": [_I, _I],
    "ic_matmul": [_P, _I, _P, _P, _I, _I, _I, _I, _I, _I, _I, _F, _P, _LL, _P],
    "ic_matmul_tune": [_P, _I, _P, _P, _I, _I, _I, _I, _I, _I, _I, _P, _LL, _P, _LL, _I, _P],
    "ic_gemm_qkv_rope_variant": [_P, _P, _P, _I, _I, _I, _I, _I, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _RF, _I, _P],
    "ic_gemm_nt_cfg": [_P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _F, _I, _I, _I, _P],
    "ic_attn_decode_splits": [_I, _I, _I, _I, _I, _I, _I, _I, _I],
    "ic_gemm_splitk_supported": [_I, _I, _I, _I, _I],
    "ic_gemm_splitk_slices": [_I, _I],
    "ic_gemm_splitk": [_P, _P, _P, _I, _I, _I, _I, _I, _I, _P],
    "ic_gemm_splitk_pays": [_I, _I, _I],
    "ic_splitk_add_rmsnorm": [_P, _I, _I, _P, _F, _P, _P, _I, _F, _P],
    "ic_rule_few_rows": [],
    "ic_rule_sumsq_parts_max": [],
    "ic_rule_own_product": [_I, _I, _I, _I],
    "ic_rule_qkv_fused": [_I, _I, _I, _I, _I, _I, _I, _I, _I],
    "ic_rule_gate_up_fused": [_I, _I, _I, _I, _I, _I],
    "ic_rule_tail": [_I, _I, _I, _I, _I, _I],
    "ic_rule_attention": [_I, _I, _I, _I, _I],
    "ic_rule_context_bucket": [_I],
    "ic_attn_decode_on_matrix_cores": [_I, _I, _I],
    "ic_decoder_create": [_c.POINTER(IcDecoderMeta), _c.POINTER(IcLayer), _c.POINTER(IcRunEntry)],
    "ic_decoder_create_error": [],
    "ic_decoder_destroy": [_P],
    "ic_decoder_last_error": [_P],
    "ic_decoder_workspace_bytes": [_P, _c.POINTER(IcStepBatch)],
    "ic_decoder_forward": [_P, _c.POINTER(IcStepBatch), _P, _LL, _P, _LL, _P, _P],
    "ic_decoder_step_ints": [_P, _c.POINTER(IcHostBatch)],
    "ic_decoder_pack": [_P, _c.POINTER(IcHostBatch), _P, _P, _LL, _c.POINTER(IcStepBatch)],
    "ic_decoder_step": [_P, _c.POINTER(IcHostBatch), _P, _P, _LL, _P, _LL, _P, _LL, _P, _c.POINTER(IcStepBatch), _P],
}
_RESTYPES = {"ic_decoder_create": _P, "ic_decoder_create_error": _c.c_char_p, "ic_decoder_destroy": None,
             "ic_decoder_last_error": _c.c_char_p, "ic_decoder_workspace_bytes": _LL, "ic_decoder_step_ints": _LL,
             "ic_peak_mfma_bf16": _LL, "ic_attn_prefill_scratch_floats": _LL}


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
                fn.restype = _RESTYPES.get(name, _I)
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
