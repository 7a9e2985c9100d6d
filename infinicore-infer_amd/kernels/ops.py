"""Python face of the HIP kernels: one function per kernel.  Each checks on the
host that shapes, dtypes and strides are what the kernel and its grid assume,
then launches on torch's current stream.  Nothing here computes on the CPU.
"""
import torch

from .lib import IcResidualNorm, IcRowFactor, KernelError, check, get_lib

F32, BF16 = 0, 1
_DT = {torch.float32: F32, torch.bfloat16: BF16}


def dtype_code(dt) -> int:
    try:
        return _DT[dt]
    except KeyError:
        raise KernelError("dtype %s is not supported by the kernels (float32, bfloat16)" % dt)


_scoped_stream = None


class stream_scope:
    """Looks torch's current stream up once and uses it for every launch inside the ``with`` block
    (the lookup costs about as much as a launch).  Do not switch streams inside the block."""

    def __enter__(self):
        global _scoped_stream
        self._outer = _scoped_stream
        _scoped_stream = torch.cuda.current_stream().cuda_stream
        return self

    def __exit__(self, *exc):
        global _scoped_stream
        _scoped_stream = self._outer
        return False


def _stream():
    return _scoped_stream if _scoped_stream is not None else torch.cuda.current_stream().cuda_stream


def current_stream():
    """The stream the kernels launch on (the scoped one inside ``stream_scope``)."""
    return _stream()


def _need(cond, what):
    if not cond:
        raise KernelError(what)


def _dev(*ts):
    for t in ts:
        if t is not None and not t.is_cuda:
            raise KernelError("kernel operands must be on the GPU (got a %s tensor)" % t.device)


def _i32(t, name):
    _need(t.dtype == torch.int32 and t.is_contiguous(), "%s must be a contiguous int32 tensor" % name)


def embed(tokens, table, out, scale: float):
    """out[t, :] = table[tokens[t], :] * scale; out is float32 [T, d]."""
    _dev(tokens, table, out)
    _i32(tokens, "tokens")
    T, d = out.shape
    _need(tokens.numel() == T and table.dim() == 2 and table.shape[1] == d, "embed: shape mismatch")
    _need(out.dtype == torch.float32 and out.is_contiguous() and table.is_contiguous(), "embed: layout")
    check(get_lib().ic_embed(tokens.data_ptr(), table.data_ptr(), dtype_code(table.dtype), out.data_ptr(),
                             T, d, float(scale), _stream()), "embed")
    return out


def rmsnorm(x, weight, out, eps: float, out_scale: float = 1.0, rows=None):
    """out[r] = x[rows[r] or r] * rsqrt(mean(x^2) + eps) * weight * out_scale.  x is float32."""
    _dev(x, weight, out, rows)
    d = x.shape[-1]
    n = out.shape[0]
    _need(x.dtype == torch.float32 and x.is_contiguous() and out.is_contiguous(), "rmsnorm: layout")
    _need(weight.dtype == torch.float32 and weight.numel() == d and out.shape[-1] == d, "rmsnorm: shape mismatch")
    if rows is not None:
        _i32(rows, "rows")
        _need(rows.numel() == n, "rmsnorm: rows/out mismatch")
    else:
        _need(x.shape[0] == n, "rmsnorm: x/out mismatch")
    check(get_lib().ic_rmsnorm(x.data_ptr(), rows.data_ptr() if rows is not None else None, weight.data_ptr(),
                               out.data_ptr(), dtype_code(out.dtype), n, d, float(eps), float(out_scale),
                               _stream()), "rmsnorm")
    return out


def add_rmsnorm(x, y, alpha: float, weight, out, eps: float):
    """x += alpha * y (x float32, in place); out = rmsnorm(x) * weight."""
    _dev(x, y, weight, out)
    T, d = x.shape
    _need(x.dtype == torch.float32 and x.is_contiguous() and y.is_contiguous() and out.is_contiguous(),
          "add_rmsnorm: layout")
    _need(tuple(y.shape) == (T, d) and tuple(out.shape) == (T, d) and weight.numel() == d
          and weight.dtype == torch.float32, "add_rmsnorm: shape mismatch")
    check(get_lib().ic_add_rmsnorm(x.data_ptr(), y.data_ptr(), dtype_code(y.dtype), float(alpha),
                                   weight.data_ptr(), out.data_ptr(), dtype_code(out.dtype), T, d,
                                   float(eps), _stream()), "add_rmsnorm")
    return out


def residual_add(x, y, alpha: float):
    """x += alpha * y; x float32."""
    _dev(x, y)
    _need(x.dtype == torch.float32 and x.is_contiguous() and y.is_contiguous() and x.shape == y.shape,
          "residual_add: layout")
    check(get_lib().ic_residual_add(x.data_ptr(), y.data_ptr(), dtype_code(y.dtype), float(alpha),
                                    x.numel(), _stream()), "residual_add")
    return x


def swiglu(gate_up, out):
    """out[t, j] = up * silu(gate), gate = gate_up[t, j], up = gate_up[t, di + j]."""
    _dev(gate_up, out)
    T, di = out.shape
    _need(tuple(gate_up.shape) == (T, 2 * di) and gate_up.is_contiguous() and out.is_contiguous()
          and gate_up.dtype == out.dtype, "swiglu: layout")
    check(get_lib().ic_swiglu(gate_up.data_ptr(), out.data_ptr(), dtype_code(out.dtype), T, di, _stream()),
          "swiglu")
    return out


def copy_pages(planes, src, dst):
    """planes[..., dst[i], :, :, :] = planes[..., src[i], :, :, :] for a cache group's planes
    [slots, planes, pages, kv_heads, page_size, head_dim] (contiguous); src, dst: int32 page ids on the device."""
    _dev(planes, src, dst)
    _i32(src, "src")
    _i32(dst, "dst")
    _need(planes.dim() == 6 and planes.is_contiguous() and src.numel() == dst.numel(), "copy_pages: layout")
    n_pages = planes.shape[2]
    page_bytes = planes.shape[3] * planes.shape[4] * planes.shape[5] * planes.element_size()
    check(get_lib().ic_copy_pages(planes.data_ptr(), planes.shape[0] * planes.shape[1], n_pages, page_bytes,
                                  src.data_ptr(), dst.data_ptr(), src.numel(), _stream()), "copy_pages")


def rope_kv_write(qkv, positions, cos, sin, kcache, vcache, slots, n_heads, n_kv_heads, head_dim,
                  rot_dim, page_size):
    """Rotate the q heads of qkv[T, H] in place; rotate the k heads and copy the
    v heads into cache slot ``slots[t]``.  n_kv_heads == 0: q only, no cache write."""
    _dev(qkv, positions, cos, sin, kcache, vcache, slots)
    T = qkv.shape[0]
    _i32(positions, "positions")
    _need(qkv.dim() == 2 and qkv.stride(1) == 1, "rope: qkv must be [T, H] with unit inner stride")
    _need(qkv.shape[1] >= (n_heads + 2 * n_kv_heads) * head_dim, "rope: qkv row too short")
    _need(positions.numel() == T, "rope: positions/qkv mismatch")
    half = rot_dim // 2
    if rot_dim > 0:
        _need(cos.dtype == torch.float32 and sin.dtype == torch.float32 and cos.is_contiguous()
              and sin.is_contiguous() and cos.shape[-1] == half and sin.shape == cos.shape,
              "rope: cos/sin must be float32 [max_pos, rot/2]")
    if n_kv_heads > 0:
        _i32(slots, "slots")
        _need(slots.numel() == T, "rope: slots/qkv mismatch")
        _need(kcache.dtype == qkv.dtype and vcache.dtype == qkv.dtype, "rope: cache dtype differs from qkv")
        _need(kcache.is_contiguous() and vcache.is_contiguous()
              and tuple(kcache.shape[1:]) == (n_kv_heads, page_size, head_dim)
              and kcache.shape == vcache.shape, "rope: cache must be [pages, kv_heads, page_size, head_dim]")
    check(get_lib().ic_rope_kv_write(
        qkv.data_ptr(), dtype_code(qkv.dtype), positions.data_ptr(),
        cos.data_ptr() if rot_dim > 0 else None, sin.data_ptr() if rot_dim > 0 else None,
        kcache.data_ptr() if n_kv_heads > 0 else None, vcache.data_ptr() if n_kv_heads > 0 else None,
        slots.data_ptr() if n_kv_heads > 0 else None,
        T, qkv.stride(0), n_heads, n_kv_heads, head_dim, rot_dim, page_size, _stream()), "rope_kv_write")


def _attn_common(q, out, kcache, vcache, block_tables, n_heads, n_kv_heads, head_dim, page_size):
    _dev(q, out, kcache, vcache, block_tables)
    _need(q.dim() == 2 and q.stride(1) == 1 and q.shape[1] >= n_heads * head_dim, "attention: q layout")
    _need(out.dim() == 2 and out.stride(1) == 1 and out.shape[1] >= n_heads * head_dim, "attention: out layout")
    _need(q.dtype == out.dtype == kcache.dtype == vcache.dtype, "attention: dtypes differ")
    _need(kcache.is_contiguous() and vcache.is_contiguous() and kcache.shape == vcache.shape
          and tuple(kcache.shape[1:]) == (n_kv_heads, page_size, head_dim),
          "attention: cache must be [pages, kv_heads, page_size, head_dim]")
    _need(block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.stride(1) == 1,
          "attention: block_tables must be int32 [R, max_blocks]")
    _need(n_heads % n_kv_heads == 0, "attention: heads not a multiple of kv heads")


def attention_generic(q, out, kcache, vcache, block_tables, token_req, positions, n_heads, n_kv_heads,
                      head_dim, page_size, scale: float, window: int = 0):
    """out[t, h] = softmax over keys <= positions[t] (within the window) of q[t, h] . K, times V."""
    _attn_common(q, out, kcache, vcache, block_tables, n_heads, n_kv_heads, head_dim, page_size)
    _i32(token_req, "token_req")
    _i32(positions, "positions")
    T = q.shape[0]
    _need(token_req.numel() == T and positions.numel() == T and out.shape[0] == T, "attention: T mismatch")
    _need(head_dim <= 512, "attention: head size above 512")
    check(get_lib().ic_attn_generic(
        q.data_ptr(), q.stride(0), out.data_ptr(), out.stride(0), dtype_code(q.dtype), kcache.data_ptr(),
        vcache.data_ptr(), block_tables.data_ptr(), block_tables.stride(0), token_req.data_ptr(),
        positions.data_ptr(), T, n_heads, n_kv_heads, head_dim, page_size, float(scale), int(window or 0),
        _stream()), "attention_generic")


def attention_decode_supported(dtype, head_dim: int) -> bool:
    return bool(get_lib().ic_attn_decode_supported(dtype_code(dtype), head_dim))


def attention_decode_on_matrix_cores(dtype, n_heads: int, n_kv_heads: int) -> bool:
    """True when attention_decode runs its grouped-query kernel (bfloat16, several query heads per
    kv head): that kernel wants fewer key splits than the one-head-per-wave kernel (the library's rule)."""
    return bool(get_lib().ic_attn_decode_on_matrix_cores(dtype_code(dtype), int(n_heads), int(n_kv_heads)))


def attention_decode_splits(n_rows: int, n_heads: int, n_kv_heads: int, head_dim: int, elem_bytes: int, window: int,
                            max_context: int, matrix_cores: int, compute_units: int) -> int:
    """Ways to split the keys of ``n_rows`` single-token rows that see up to ``max_context`` keys (the library's
    cost model of its two kernels, fitted to sweeps)."""
    return int(get_lib().ic_attn_decode_splits(int(n_rows), int(n_heads), int(n_kv_heads), int(head_dim), int(elem_bytes),
                                               int(window or 0), int(max_context), int(bool(matrix_cores)),
                                               int(compute_units)))


def attention_decode(q, out, kcache, vcache, block_tables, tok_list, n_tok, token_req, positions, part_acc,
                     part_ml, n_heads, n_kv_heads, head_dim, page_size, scale: float, window: int, n_split: int):
    """Split-key attention of the single tokens listed in tok_list (None: rows 0..n_tok-1)."""
    _attn_common(q, out, kcache, vcache, block_tables, n_heads, n_kv_heads, head_dim, page_size)
    _i32(token_req, "token_req")
    _i32(positions, "positions")
    if tok_list is not None:
        _i32(tok_list, "tok_list")
        _need(tok_list.numel() >= n_tok, "attention_decode: tok_list too short")
    else:
        _need(q.shape[0] >= n_tok, "attention_decode: fewer rows than tokens")
    _need(part_acc.dtype == torch.float32 and part_acc.is_contiguous()
          and part_acc.numel() >= n_tok * n_heads * n_split * head_dim, "attention_decode: part_acc too small")
    _need(part_ml.dtype == torch.float32 and part_ml.is_contiguous()
          and part_ml.numel() >= n_tok * n_heads * n_split * 2, "attention_decode: part_ml too small")
    check(get_lib().ic_attn_decode(
        q.data_ptr(), q.stride(0), out.data_ptr(), out.stride(0), dtype_code(q.dtype), kcache.data_ptr(),
        vcache.data_ptr(), block_tables.data_ptr(), block_tables.stride(0),
        tok_list.data_ptr() if tok_list is not None else None, token_req.data_ptr(), positions.data_ptr(),
        part_acc.data_ptr(), part_ml.data_ptr(), n_tok, n_heads, n_kv_heads, head_dim, page_size,
        float(scale), int(window or 0), int(n_split), _stream()), "attention_decode")


def attention_prefill_supported(dtype, head_dim: int, page_size: int) -> bool:
    return bool(get_lib().ic_attn_prefill_supported(dtype_code(dtype), head_dim, page_size))


def attention_prefill_tile_rows() -> int:
    return get_lib().ic_attn_prefill_tile_rows()


def attention_prefill_parts(n_tiles: int, n_heads: int, head_dim: int, max_keys: int, compute_units: int):
    """(parts, part_len): into how many blocks of their own to cut the query tiles' walks over the keys when the longest
    tile of the step sees ``max_keys`` keys (1: no cut), and how many key tiles of 64 a part holds at least."""
    import ctypes
    part_len = ctypes.c_int(0)
    parts = get_lib().ic_attn_prefill_parts(int(n_tiles), int(n_heads), int(head_dim), int(max_keys), int(compute_units),
                                            ctypes.byref(part_len))
    return int(parts), int(part_len.value)


def attention_prefill_parts_of_step(dtype, n_tiles: int, n_heads: int, head_dim: int, max_position: int, window: int, compute_units: int):
    """(parts, part_len) for a step whose largest position is ``max_position`` under a mixer's ``window`` (0: none);
    float32 walks are never cut."""
    import ctypes
    part_len = ctypes.c_int(0)
    parts = get_lib().ic_attn_prefill_parts_of_step(dtype_code(dtype), int(n_tiles), int(n_heads), int(head_dim), int(max_position), int(window or 0),
                                                    int(compute_units), ctypes.byref(part_len))
    return int(parts), int(part_len.value)


def attention_prefill_counter_ints() -> int:
    return int(get_lib().ic_attn_prefill_counter_ints())


def attention_prefill_scratch_floats(n_tiles: int, n_heads: int, head_dim: int, parts: int) -> int:
    return int(get_lib().ic_attn_prefill_scratch_floats(int(n_tiles), int(n_heads), int(head_dim), int(parts)))


def attention_prefill(q, out, kcache, vcache, block_tables, tiles, n_tiles, n_heads, n_kv_heads, head_dim,
                      page_size, scale: float, window: int = 0, groups: int = 0, parts: int = 1, part_len: int = 0,
                      scratch=None, counters=None):
    """Matrix-core attention of prompt portions.  tiles: int32 [n, 4] rows of
    (request row in block_tables, first token row, rows <= tile_rows, first position).
    groups: wave groups per query tile (1 or 2); 0 lets the kernel choose from the number of blocks.
    parts > 1: every tile's walk over the keys is cut into up to ``parts`` blocks of at least ``part_len`` key tiles
    that meet through ``scratch`` (float32, attention_prefill_scratch_floats(...) elements) and count themselves in at
    ``counters`` (int32, attention_prefill_counter_ints() elements, zero before the first launch; every launch leaves them
    zero; launches that overlap in time need counters of their own)."""
    _need(groups in (0, 1, 2), "attention_prefill: groups must be 0, 1 or 2")
    _attn_common(q, out, kcache, vcache, block_tables, n_heads, n_kv_heads, head_dim, page_size)
    _need(tiles.dtype == torch.int32 and tiles.is_contiguous() and tiles.dim() == 2 and tiles.shape[1] == 4
          and tiles.shape[0] >= n_tiles, "attention_prefill: tiles must be int32 [n, 4]")
    if parts > 1:
        _dev(scratch)
        _dev(counters)
        _need(scratch is not None and scratch.dtype == torch.float32 and scratch.is_contiguous(),
              "attention_prefill: a cut walk needs float32 scratch memory")
        _need(counters is not None and counters.dtype == torch.int32 and counters.is_contiguous()
              and counters.numel() >= attention_prefill_counter_ints(), "attention_prefill: a cut walk needs its int32 arrival counters")
    check(get_lib().ic_attn_prefill_split(
        q.data_ptr(), q.stride(0), out.data_ptr(), out.stride(0), dtype_code(q.dtype), kcache.data_ptr(),
        vcache.data_ptr(), block_tables.data_ptr(), block_tables.stride(0), tiles.data_ptr(), n_tiles,
        n_heads, n_kv_heads, head_dim, page_size, float(scale), int(window or 0), int(groups), int(parts), int(part_len),
        scratch.data_ptr() if parts > 1 else None, scratch.numel() if parts > 1 else 0,
        counters.data_ptr() if parts > 1 else None, _stream()),
        "attention_prefill")


def sample(logits, out, temperature=None, top_k=None, top_p=None, uniform=None):
    """out[r] = token sampled from logits[r] (float32 [R, V]).  temperature None: argmax."""
    _dev(logits, out, temperature, top_k, top_p, uniform)
    R, V = logits.shape
    _need(logits.dtype == torch.float32 and logits.stride(1) == 1, "sample: logits must be float32 rows")
    _i32(out, "out")
    _need(out.numel() >= R, "sample: out too short")
    if temperature is not None:
        _need(temperature.dtype == torch.float32 and top_p.dtype == torch.float32
              and uniform.dtype == torch.float32 and top_k.dtype == torch.int32, "sample: parameter dtypes")
        _need(min(temperature.numel(), top_k.numel(), top_p.numel(), uniform.numel()) >= R,
              "sample: parameter arrays too short")
    p = lambda t: t.data_ptr() if t is not None else None
    check(get_lib().ic_sample(logits.data_ptr(), logits.stride(0), R, V, p(temperature), p(top_k), p(top_p),
                              p(uniform), out.data_ptr(), _stream()), "sample")
    return out


def argmax(logits, out, scratch_val, scratch_idx):
    """out[r] = index of the largest logit of row r (the lowest index among equals), in two
    stages; scratch_val float32 and scratch_idx int32 of at least 64 * rows elements."""
    _dev(logits, out, scratch_val, scratch_idx)
    R, V = logits.shape
    _need(logits.dtype == torch.float32 and logits.stride(1) == 1, "argmax: logits must be float32 rows")
    _i32(out, "out")
    _i32(scratch_idx, "scratch_idx")
    _need(out.numel() >= R and scratch_val.dtype == torch.float32 and scratch_val.is_contiguous()
          and scratch_val.numel() >= 64 * R and scratch_idx.numel() >= 64 * R, "argmax: buffers too small")
    check(get_lib().ic_argmax(logits.data_ptr(), logits.stride(0), R, V, scratch_val.data_ptr(),
                              scratch_idx.data_ptr(), out.data_ptr(), _stream()), "argmax")
    return out


def argmax_static(logits, out):
    """argmax with the library's own static scratch memory: allocates nothing, takes at most
    ``get_lib().ic_argmax_static_max_rows()`` rows; calls that overlap on one GPU race."""
    _dev(logits, out)
    R, V = logits.shape
    _need(logits.dtype == torch.float32 and logits.stride(1) == 1, "argmax_static: logits must be float32 rows")
    _i32(out, "out")
    _need(out.numel() >= R, "argmax_static: out too short")
    check(get_lib().ic_argmax_static(logits.data_ptr(), logits.stride(0), R, V, out.data_ptr(), _stream()),
          "argmax_static")
    return out


def gemm_nt_supported(a_dtype, w_dtype, c_dtype) -> bool:
    try:
        return bool(get_lib().ic_gemm_nt_supported(dtype_code(a_dtype), dtype_code(w_dtype), dtype_code(c_dtype)))
    except KernelError:
        return False


# ---- which kernel takes what: the library's rules, shared with its native step function ----------------------------
TAIL_PLAIN, TAIL_SPLIT_NORM, TAIL_SLICES = 0, 1, 2
ATTN_GENERAL, ATTN_SINGLE_TOKENS, ATTN_PORTIONS = 0, 1, 2


def _code_or_none(dt):
    return _DT.get(dt)


def rule_own_product(a_dtype, w_dtype, c_dtype, rows: int) -> bool:
    """True when a plain product of ``rows`` rows runs in the package's own kernel (gemm_nt), not in the library."""
    codes = (_code_or_none(a_dtype), _code_or_none(w_dtype), _code_or_none(c_dtype))
    return None not in codes and bool(get_lib().ic_rule_own_product(codes[0], codes[1], codes[2], int(rows)))


def rule_qkv_fused(dtype, rows: int, a, w, head_dim: int, rot_dim: int, kv_heads_written: int, row_factors_owed: bool) -> bool:
    """True when the QKV projection of a[rows, K] with w runs with rotary and cache write in its epilogue."""
    code = _code_or_none(dtype)
    return code is not None and bool(get_lib().ic_rule_qkv_fused(code, int(rows), int(a.shape[1]), int(a.stride(0)), int(w.stride(0)),
                                                                 int(head_dim), int(rot_dim), int(kv_heads_written),
                                                                 int(bool(row_factors_owed))))


def rule_gate_up_fused(dtype, rows: int, a, w, row_factors_owed: bool) -> bool:
    """True when the gate/up projection of a[rows, K] with w runs with SwiGLU in its epilogue."""
    code = _code_or_none(dtype)
    return code is not None and bool(get_lib().ic_rule_gate_up_fused(code, int(rows), int(a.shape[1]), int(a.stride(0)),
                                                                     int(w.stride(0)), int(bool(row_factors_owed))))


def rule_tail(dtype, a, w) -> int:
    """How the projection a w^T into the residual stream, followed by a norm, runs: TAIL_PLAIN, TAIL_SPLIT_NORM or TAIL_SLICES."""
    code = _code_or_none(dtype)
    if code is None or a.dtype != dtype or w.dtype != dtype:
        return TAIL_PLAIN
    return int(get_lib().ic_rule_tail(code, int(a.shape[0]), int(w.shape[0]), int(a.shape[1]), int(a.stride(0)), int(w.stride(0))))


def rule_attention(dtype, head_dim: int, page_size: int, n_decode_rows: int, n_tiles: int) -> int:
    """ATTN_GENERAL, or the bits ATTN_SINGLE_TOKENS and ATTN_PORTIONS: which attention kernels a step takes."""
    return int(get_lib().ic_rule_attention(dtype_code(dtype), int(head_dim), int(page_size), int(n_decode_rows), int(n_tiles)))


def rule_context_bucket(n_keys: int) -> int:
    """The key count that the key split of single-token rows is chosen for (rounded up, so that a recorded step
    serves a range of lengths and splits as an eager one does)."""
    return int(get_lib().ic_rule_context_bucket(int(n_keys)))


def max_sumsq_parts() -> int:
    """Column blocks of sums of squares a product can take as row factors."""
    return int(get_lib().ic_rule_sumsq_parts_max())


def residual_parts(n: int) -> int:
    """Column blocks of sums of squares that gemm_nt(..., residual=...) writes for an n wide product."""
    return int(get_lib().ic_gemm_nt_residual_parts(int(n)))


def _row_factor(row_factor, M, what):
    """row_factor = (sumsq float32 [n_parts, 16], width, eps) -> the C struct (or None)."""
    if row_factor is None:
        return None
    sumsq, width, eps = row_factor
    _dev(sumsq)
    _need(M <= 16, what + ": row factors need at most 16 rows")
    _need(sumsq.dtype == torch.float32 and sumsq.is_contiguous() and sumsq.dim() == 2 and sumsq.shape[1] == 16
          and 0 < sumsq.shape[0] <= max_sumsq_parts(), what + ": sums of squares must be float32 [<= 256, 16]")
    _need(width > 0, what + ": width")
    return IcRowFactor(sumsq.data_ptr(), sumsq.shape[0], int(width), float(eps))


def gemm_epilogue_rows(kind: str, a, w) -> int:
    """Rows that the product with the ``kind`` epilogue ("swiglu", or "rope" for gemm_qkv_rope) takes for these operands: 32
    where the weights can be read in whole cache lines, 16 otherwise (and above 16 rows without row factors)."""
    return int(get_lib().ic_gemm_nt_epilogue_rows({"swiglu": 1, "rope": 2}[kind], int(a.shape[1]), int(a.stride(0)), int(w.stride(0))))


def gemm_nt(a, w, out, alpha: float = 1.0, swiglu_output: bool = False, row_factor=None, residual=None, whole_lines: bool = True):
    """out[M, N] = alpha * a[M, K] @ w[N, K]^T (bfloat16 operands, float32 accumulation).
    swiglu_output (M <= gemm_epilogue_rows("swiglu", a, w)): w = [gate rows; up rows] and out[M, N/2] = up * silu(gate).
    row_factor = (sumsq [n_parts, 16], width, eps), M <= 16: row m of the product is first multiplied by
    rsqrt(sumsq[:, m].sum() / width + eps), the factor an RMS norm of a's rows still owes.
    residual = (x float32 [M, N], weight float32 [N], beta, sumsq_out float32 [residual_parts(N), 16]),
    M <= 16, bfloat16 out: x += beta * (the product rounded to bfloat16); out = x * weight;
    sumsq_out[b, m] = sum of x[m]^2 over columns 16 b .. 16 b + 15.
    whole_lines False (tests): the weights are loaded in operand layout also where whole cache lines would apply."""
    import ctypes
    _dev(a, w, out)
    M, K = a.shape
    N = w.shape[0]
    _need(w.shape[1] == K and tuple(out.shape) == (M, N // 2 if swiglu_output else N), "gemm_nt: shape mismatch")
    _need(not swiglu_output or (M <= 32 and N % 2 == 0), "gemm_nt: fused activation needs M <= 32 and even N")
    _need(a.stride(1) == 1 and w.stride(1) == 1 and out.stride(1) == 1, "gemm_nt: inner strides must be 1")
    rf = _row_factor(row_factor, M, "gemm_nt")
    rn = None
    mode = 1 if swiglu_output else 0
    if residual is not None:
        x, weight, beta, sumsq_out = residual
        _dev(x, weight, sumsq_out)
        _need(not swiglu_output and M <= 16 and out.dtype == torch.bfloat16, "gemm_nt: residual epilogue needs M <= 16 and bfloat16 out")
        _need(x.dtype == torch.float32 and tuple(x.shape) == (M, N) and x.stride(1) == 1, "gemm_nt: residual stream must be float32 [M, N]")
        _need(weight.dtype == torch.float32 and weight.is_contiguous() and weight.numel() == N, "gemm_nt: norm weight must be float32 [N]")
        _need(sumsq_out.dtype == torch.float32 and sumsq_out.is_contiguous()
              and tuple(sumsq_out.shape) == (residual_parts(N), 16) and residual_parts(N) <= max_sumsq_parts(),
              "gemm_nt: sumsq_out must be float32 [residual_parts(N) <= 256, 16]")
        rn = IcResidualNorm(x.data_ptr(), x.stride(0), weight.data_ptr(), float(beta), sumsq_out.data_ptr(), sumsq_out.shape[0])
        mode = 2
    if not whole_lines:
        check(get_lib().ic_gemm_nt_variant(a.data_ptr(), dtype_code(a.dtype), w.data_ptr(), dtype_code(w.dtype),
                                           out.data_ptr(), dtype_code(out.dtype), M, N, K, a.stride(0), w.stride(0),
                                           out.stride(0), float(alpha), mode, ctypes.byref(rf) if rf else None,
                                           ctypes.byref(rn) if rn else None, 0, _stream()), "gemm_nt")
        return out
    check(get_lib().ic_gemm_nt(a.data_ptr(), dtype_code(a.dtype), w.data_ptr(), dtype_code(w.dtype),
                               out.data_ptr(), dtype_code(out.dtype), M, N, K, a.stride(0), w.stride(0),
                               out.stride(0), float(alpha), mode, ctypes.byref(rf) if rf else None,
                               ctypes.byref(rn) if rn else None, _stream()), "gemm_nt")
    return out


_matmul_workspace = {}
MATMUL_WORKSPACE_BYTES = 64 << 20


def _workspace(device):
    """The library's scratch memory: one buffer per device and stream, since products that run at the
    same time on different streams must not share it (some algorithms keep flags and partial sums there)."""
    key = (device, _stream())
    ws = _matmul_workspace.get(key)
    if ws is None:
        ws = _matmul_workspace[key] = torch.empty(MATMUL_WORKSPACE_BYTES, dtype=torch.uint8, device=device)
    return ws


def library_workspace(device):
    """The library products' scratch memory for the current stream on ``device``."""
    return _workspace(device)


class NoLibraryAlgorithm(KernelError):
    """The library proposes no algorithm for a product."""


_matmul_types = {}      # (operand dtype, result dtype) -> (codes) or None: asked of the library once


def _matmul_args(a, w, out, what):
    """Checks a product's operands and returns (M, N, K, operand code, result code, row strides of a, w, out).
    Written for few attribute lookups: this runs four times a layer."""
    if not (a.is_cuda and w.is_cuda and out.is_cuda):
        _dev(a, w, out)
    M, K = a.shape
    N, Kw = w.shape
    Mo, No = out.shape
    sa, sa1 = a.stride()
    sw, sw1 = w.stride()
    so, so1 = out.stride()
    if Kw != K or Mo != M or No != N:
        raise KernelError(what + ": shape mismatch")
    if sa1 != 1 or sw1 != 1 or so1 != 1:
        raise KernelError(what + ": layout")
    key = (a.dtype, w.dtype, out.dtype)
    codes = _matmul_types.get(key, False)
    if codes is False:
        codes = None
        if a.dtype == w.dtype and a.dtype in _DT and out.dtype in _DT and \
                get_lib().ic_matmul_supported(_DT[a.dtype], _DT[out.dtype]):
            codes = (_DT[a.dtype], _DT[out.dtype])
        _matmul_types[key] = codes
    if codes is None:
        raise KernelError(what + ": unsupported types")
    return M, N, K, codes[0], codes[1], sa, sw, so


def matmul_library(a, w, out, alpha: float = 1.0):
    """out[M, N] = alpha * a[M, K] @ w[N, K]^T through the library (hipBLASLt), any number of rows.
    bfloat16 operands with a bfloat16 or float32 result, or all float32."""
    M, N, K, ca, cc, sa, sw, so = _matmul_args(a, w, out, "matmul_library")
    stream = _stream()
    ws = _matmul_workspace.get((a.device, stream))
    if ws is None:
        ws = _workspace(a.device)
    st = get_lib().ic_matmul(a.data_ptr(), ca, w.data_ptr(), out.data_ptr(), cc, M, N, K, sa, sw, so, alpha,
                        ws.data_ptr(), MATMUL_WORKSPACE_BYTES, stream)
    if st == 0:
        return out
    if st == -4:
        raise NoLibraryAlgorithm("matmul_library: no algorithm for %d x %d x %d" % (M, N, K))
    if st == -3:
        raise KernelError("matmul_library: the library refused the product %d x %d x %d" % (M, N, K))
    check(st, "matmul_library")
    return out


def matmul_library_tune(a, w, out, reps: int = 5, flush=None) -> int:
    """Times the library's algorithms for this product's shape and keeps the fastest; returns how many it tried.
    flush: a device tensor larger than the chip's caches; it is overwritten before every timed launch, so that the
    algorithms are compared with operands that come from memory, as a model's weights do."""
    M, N, K, ca, cc, sa, sw, so = _matmul_args(a, w, out, "matmul_library_tune")
    ws = _workspace(a.device)
    if flush is not None:
        _dev(a, flush)
        _need(flush.is_contiguous(), "matmul_library_tune: flush must be contiguous")
    n = get_lib().ic_matmul_tune(a.data_ptr(), ca, w.data_ptr(), out.data_ptr(), cc, M, N, K, sa, sw, so,
                                 ws.data_ptr(), ws.numel(),
                                 flush.data_ptr() if flush is not None else None,
                                 flush.numel() * flush.element_size() if flush is not None else 0, int(reps), _stream())
    if n < 0:
        raise KernelError("matmul_library_tune failed with %d for %d x %d x %d" % (n, M, N, K))
    return n


def gemm_qkv_rope_supported(dtype, head_dim: int) -> bool:
    try:
        return bool(get_lib().ic_gemm_qkv_rope_supported(dtype_code(dtype), head_dim))
    except KernelError:
        return False


def gemm_qkv_rope(a, w, qkv, positions, slots, cos, sin, kcache, vcache, n_heads, n_kv_heads, head_dim, page_size,
                  row_factor=None, tile_rows: int = 0):
    """For M <= gemm_epilogue_rows("rope", a, w) rows: qkv = a @ w^T with the rotary encoding and the cache write in the epilogue.
    The q heads of qkv[M, >= n_heads * head_dim] hold rotated queries afterwards; rotated keys and
    the values are in cache slot ``slots[m]``.  Full rotary, bfloat16.  row_factor: as in gemm_nt.
    tile_rows (tests): used weight rows per tile, 16, 8 or 4; 0: chosen from the number of heads."""
    import ctypes
    _dev(a, w, qkv, positions, slots, cos, sin, kcache, vcache)
    M, K = a.shape
    _i32(positions, "positions")
    _i32(slots, "slots")
    _need(M <= 32 and positions.numel() == M and slots.numel() == M, "gemm_qkv_rope: at most 32 rows, one position and slot each")
    rf = _row_factor(row_factor, M, "gemm_qkv_rope")
    _need(tuple(w.shape) == ((n_heads + 2 * n_kv_heads) * head_dim, K), "gemm_qkv_rope: weight shape")
    _need(qkv.shape[0] == M and qkv.shape[1] >= n_heads * head_dim and qkv.stride(1) == 1
          and a.stride(1) == 1 and w.stride(1) == 1, "gemm_qkv_rope: layout")
    _need(a.dtype == w.dtype == qkv.dtype == kcache.dtype == vcache.dtype == torch.bfloat16, "gemm_qkv_rope: bfloat16 only")
    _need(cos.dtype == torch.float32 and sin.dtype == torch.float32 and cos.is_contiguous() and sin.is_contiguous()
          and cos.shape[-1] == head_dim // 2 and sin.shape == cos.shape, "gemm_qkv_rope: cos/sin must be float32 [max_pos, dh/2]")
    _need(kcache.is_contiguous() and vcache.is_contiguous() and kcache.shape == vcache.shape
          and tuple(kcache.shape[1:]) == (n_kv_heads, page_size, head_dim), "gemm_qkv_rope: cache layout")
    args = (a.data_ptr(), w.data_ptr(), qkv.data_ptr(), M, K, a.stride(0), w.stride(0), qkv.stride(0), positions.data_ptr(),
            slots.data_ptr(), cos.data_ptr(), sin.data_ptr(), kcache.data_ptr(), vcache.data_ptr(), n_heads, n_kv_heads,
            head_dim, page_size, ctypes.byref(rf) if rf else None)
    if tile_rows:
        check(get_lib().ic_gemm_qkv_rope_variant(*args, int(tile_rows), _stream()), "gemm_qkv_rope")
    else:
        check(get_lib().ic_gemm_qkv_rope(*args, _stream()), "gemm_qkv_rope")
    return qkv


# ---- products of 17..64 rows as slices over K, and what follows them -------------------------------------------
def gemm_splitk_supported(a, w) -> bool:
    return bool(a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and a.dim() == 2 and w.dim() == 2
                and a.stride(1) == 1 and w.stride(1) == 1 and a.shape[1] == w.shape[1]
                and get_lib().ic_gemm_splitk_supported(a.shape[0], w.shape[0], a.shape[1], a.stride(0), w.stride(0)))


def gemm_splitk_pays(m: int, n: int, k: int) -> bool:
    """True when the sliced product beats the library's for an m x n x k product (17..64 rows, enough blocks)."""
    return bool(get_lib().ic_gemm_splitk_pays(int(m), int(n), int(k)))


def gemm_splitk_slices(n: int, k: int) -> int:
    return int(get_lib().ic_gemm_splitk_slices(int(n), int(k)))


def gemm_splitk(a, w, parts, n_slices=None):
    """parts[s, m, n] (float32) = a[m, K_s] . w[n, K_s] for the slices K_s of K; 1..64 rows, bfloat16 operands.
    ``parts`` must hold n_slices * M * N floats; returns its [n_slices, M, N] view."""
    _dev(a, w, parts)
    M, K = a.shape
    N = w.shape[0]
    _need(gemm_splitk_supported(a, w), "gemm_splitk: at most 64 bfloat16 rows, K a multiple of 8, rows 16-byte aligned")
    S = int(n_slices) if n_slices else gemm_splitk_slices(N, K)
    _need(parts.dtype == torch.float32 and parts.is_contiguous() and parts.numel() >= S * M * N, "gemm_splitk: parts too small")
    check(get_lib().ic_gemm_splitk(a.data_ptr(), w.data_ptr(), parts.data_ptr(), M, N, K, a.stride(0), w.stride(0), S, _stream()),
          "gemm_splitk")
    return parts.view(-1)[:S * M * N].view(S, M, N)


def splitk_add_rmsnorm(parts, x, alpha: float, weight, out, eps: float):
    """x += alpha * (the product given as slices parts [S, M, d], rounded to bfloat16); out = rmsnorm(x) * weight."""
    _dev(parts, x, weight, out)
    S, M, d = parts.shape
    _need(parts.dtype == torch.float32 and parts.is_contiguous() and x.dtype == torch.float32 and x.is_contiguous()
          and tuple(x.shape) == (M, d) and weight.dtype == torch.float32 and weight.numel() == d and weight.is_contiguous()
          and out.dtype == torch.bfloat16 and out.is_contiguous() and tuple(out.shape) == (M, d), "splitk_add_rmsnorm: layout")
    check(get_lib().ic_splitk_add_rmsnorm(parts.data_ptr(), S, M, x.data_ptr(), float(alpha), weight.data_ptr(), out.data_ptr(),
                                          d, float(eps), _stream()), "splitk_add_rmsnorm")
    return out
