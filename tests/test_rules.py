"""Which kernel takes what: the kernel library's dispatch rules, asked the way the parts' Python forward and the
native step function ask them.  The functions are host code, so they are tested without a GPU (with no device to
ask, the library assumes 256 compute units).  (CPU)"""
import torch

BF16, F32 = torch.bfloat16, torch.float32


def _ops():
    from infinicore_infer_amd.kernels import ops
    return ops


class _Mat:
    """Stands in for a tensor where a rule only reads shape, stride and dtype."""

    def __init__(self, rows, cols, dtype=BF16, stride=None):
        self.shape, self.dtype, self._stride = (rows, cols), dtype, stride or cols

    def stride(self, i):
        return self._stride if i == 0 else 1


def test_key_counts_are_rounded_up_for_the_split_choice():
    ops = _ops()
    assert [ops.rule_context_bucket(n) for n in (1, 256, 257, 1024)] == [256, 256, 512, 1024]
    # above 1,024 keys: multiples of a quarter of the power of two below
    assert [ops.rule_context_bucket(n) for n in (1025, 2049, 2560, 2561, 4097, 16400)] == [1280, 2560, 2560, 3072, 5120, 20480]
    for n in range(1, 40000, 37):
        b = ops.rule_context_bucket(n)
        assert n <= b <= (max(256, 2 * n) if n <= 1024 else int(1.25 * n) + 1)


def test_products_of_a_layer_at_the_benchmark_sizes():
    ops = _ops()
    d, di = 2304, 5760
    for rows, own in ((1, True), (16, True), (17, False), (2048, False)):
        assert ops.rule_own_product(BF16, BF16, BF16, rows) == own
        assert ops.rule_own_product(BF16, BF16, F32, rows) == own          # the head writes float32 logits
    assert not ops.rule_own_product(F32, F32, F32, 1)                       # the 32-bit path: the library's true-float32 product
    w_qkv, w_gu = _Mat(3 * d, d), _Mat(2 * di, d)
    # QKV with rotary and cache write, gate/up with SwiGLU: up to 16 rows always, up to 32 with whole-line weight loads
    # (K a multiple of 64) unless half-normed rows are owed
    for rows, owed, fused in ((1, True, True), (16, True, True), (17, True, False), (17, False, True), (32, False, True), (33, False, False)):
        assert ops.rule_qkv_fused(BF16, rows, _Mat(rows, d), w_qkv, 64, 64, 36, owed) == fused
        assert ops.rule_gate_up_fused(BF16, rows, _Mat(rows, d), w_gu, owed) == fused
    assert not ops.rule_qkv_fused(BF16, 8, _Mat(8, d), w_qkv, 64, 32, 36, False)      # partial rotary: the rotary kernel
    assert not ops.rule_qkv_fused(BF16, 8, _Mat(8, d), w_qkv, 64, 64, 0, False)       # an entry that writes no cache
    assert not ops.rule_qkv_fused(F32, 8, _Mat(8, d, F32), _Mat(3 * d, d, F32), 64, 64, 36, False)
    assert not ops.rule_qkv_fused(BF16, 20, _Mat(20, 200), _Mat(600, 200), 64, 64, 2, False)     # K no multiple of 64: 16 rows at most
    assert ops.rule_qkv_fused(BF16, 16, _Mat(16, 200), _Mat(600, 200), 64, 64, 2, False)
    # the projections into the residual stream: the norm split over the products up to 16 rows, slices over K up to 64, else plain
    for rows, how in ((1, ops.TAIL_SPLIT_NORM), (16, ops.TAIL_SPLIT_NORM), (17, ops.TAIL_SLICES), (64, ops.TAIL_SLICES), (65, ops.TAIL_PLAIN)):
        assert ops.rule_tail(BF16, _Mat(rows, d), _Mat(d, d)) == how            # O
        assert ops.rule_tail(BF16, _Mat(rows, di), _Mat(d, di)) == how          # down
    assert ops.rule_tail(F32, _Mat(4, d, F32), _Mat(d, d, F32)) == ops.TAIL_PLAIN
    assert ops.rule_tail(BF16, _Mat(4, d), _Mat(d, d, F32)) == ops.TAIL_PLAIN     # a matrix stored in 32-bit
    # 13..16 rows of 16 KB and more (the 8B shape's down projection) already run as slices
    assert ops.rule_tail(BF16, _Mat(14, 16384), _Mat(4096, 16384)) == ops.TAIL_SLICES
    assert ops.rule_tail(BF16, _Mat(12, 16384), _Mat(4096, 16384)) == ops.TAIL_SPLIT_NORM
    # a small model: too few blocks for slices to pay
    assert ops.rule_tail(BF16, _Mat(20, 64), _Mat(64, 64)) == ops.TAIL_PLAIN


def test_attention_kernels_of_a_step():
    ops = _ops()
    both = ops.ATTN_SINGLE_TOKENS | ops.ATTN_PORTIONS
    for dtype in (BF16, F32):
        assert ops.rule_attention(dtype, 64, 64, 8, 0) == ops.ATTN_SINGLE_TOKENS
        assert ops.rule_attention(dtype, 128, 16, 0, 5) == ops.ATTN_PORTIONS
        assert ops.rule_attention(dtype, 64, 32, 50, 2) == both
        assert ops.rule_attention(dtype, 80, 64, 3, 2) == ops.ATTN_GENERAL        # a head size without tiled kernels
        assert ops.rule_attention(dtype, 64, 48, 3, 2) == ops.ATTN_GENERAL        # pages that are no power of two: one kernel for all rows
        assert ops.rule_attention(dtype, 64, 48, 3, 0) == ops.ATTN_SINGLE_TOKENS  # (single tokens alone do not mind)
    assert ops.attention_decode_on_matrix_cores(BF16, 24, 8) and not ops.attention_decode_on_matrix_cores(BF16, 36, 36)
    assert not ops.attention_decode_on_matrix_cores(F32, 24, 8)
    # the walks of prompt tiles: cut for few blocks and long walks in bfloat16, never in float32
    assert ops.attention_prefill_parts_of_step(BF16, 16, 36, 64, 2047, 0, 256) == (2, 16)
    assert ops.attention_prefill_parts_of_step(F32, 16, 36, 64, 2047, 0, 256)[0] == 1
    assert ops.attention_prefill_parts_of_step(BF16, 4, 36, 64, 4095, 512, 256)[0] == 1      # a window of 512 keys: short walks
    # the key split of single tokens: never for short contexts, several for few rows over long ones
    assert ops.attention_decode_splits(8, 36, 36, 64, 2, 0, 256, 0, 256) == 1
    assert ops.attention_decode_splits(1, 36, 36, 64, 2, 0, 16384, 0, 256) > 4
    assert ops.attention_decode_splits(64, 36, 36, 64, 2, 0, 2560, 0, 256) == 1


def test_cut_walks_of_prompt_tiles():
    """How a step's prompt tiles are cut: (tiles, heads, head size, keys the longest tile sees, compute units) -> (parts, key
    tiles a part)."""
    ops = _ops()
    parts = ops.attention_prefill_parts
    assert parts(16, 36, 64, 2048, 256) == (2, 16)          # the benchmark's prompt: 576 blocks of 32 key tiles
    assert parts(32, 36, 64, 4096, 256)[0] == 1             # many blocks: left whole
    assert parts(16, 32, 128, 2048, 256)[0] == 1            # two blocks a unit at head size 128: two wave groups do it
    assert parts(4, 40, 128, 4096, 256) == (3, 22)
    # few blocks (a portion or two beside decoded tokens): shorter walks are cut too
    assert parts(4, 36, 64, 2048, 256) == (3, 11) and parts(4, 24, 64, 1024, 256) == (3, 6) and parts(2, 24, 64, 1280, 256) == (4, 5)
    assert parts(4, 24, 64, 704, 256)[0] == 1 and parts(4, 36, 64, 1024, 256)[0] == 1
    assert parts(4, 32, 128, 1024, 256) == (2, 8) and parts(2, 32, 128, 1280, 256) == (4, 5) and parts(8, 32, 128, 1024, 256)[0] == 1
    # a part never has fewer key tiles than the rule's least, and the parts cover the walk
    for tiles in (1, 2, 4, 8, 16):
        for heads, dh in ((8, 64), (24, 64), (36, 64), (32, 128), (2, 128)):
            for keys in range(64, 8200, 448):
                p, n = parts(tiles, heads, dh, keys, 256)
                longest = (keys + 63) // 64
                assert 1 <= p <= 4 and p * n >= longest and (p == 1 or n >= 4)
    # the scratch memory the parts need
    assert ops.attention_prefill_scratch_floats(4, 36, 64, 4) == 4 * 36 * 4 * 256 * 34 and ops.attention_prefill_scratch_floats(4, 36, 64, 1) == 0

