"""Each HIP kernel alone against a plain float64 reference of the same op, at
sizes other than the tiny models': widths and vocabularies that are no power of
two, head sizes in steps of 16, odd numbers of heads and groups."""
import math

import pytest
import torch

import plain_model as P

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
DT = [torch.float32, torch.bfloat16]


def _ops():
    from infinicore_infer_amd.kernels import ops
    return ops


def _tol(dtype):
    return 2e-6 if dtype == torch.float32 else 1e-2


def _close(got, want, dtype, scale=None, factor=1.0):
    got, want = got.double().cpu(), want.double().cpu()
    s = float(want.abs().max()) if scale is None else scale
    err = float((got - want).abs().max()) / max(s, 1e-30)
    assert math.isfinite(err) and err <= _tol(dtype) * factor, "error %.3g of the largest value" % err


# ---------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("T,d,V", [(1, 64, 50), (37, 200, 331), (300, 2304, 1000)])
def test_embed(dtype, T, d, V):
    g = torch.Generator().manual_seed(1)
    table = torch.randn(V, d, generator=g).to(dtype)
    tok = torch.randint(0, V, (T,), generator=g, dtype=torch.int32)
    out = torch.empty(T, d, device=DEV)
    _ops().embed(tok.to(DEV), table.to(DEV), out, 12.0)
    want = P.plain_embedding(table, tok.tolist(), 12.0)
    _close(out, want, torch.float32)


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("T,d,eps", [(1, 64, 1e-5), (33, 200, 1e-6), (17, 2304, 1e-5), (5, 4097, 1e-2),
                                     (2051, 200, 1e-5), (1027, 5000, 1e-5)])     # many rows
def test_rmsnorm(dtype, T, d, eps):
    g = torch.Generator().manual_seed(2)
    x = torch.randn(T, d, generator=g) * 3
    x[0] *= 1e-3                      # a tiny row: eps inside the root matters there
    w = 1 + 0.1 * torch.randn(d, generator=g)
    out = torch.empty(T, d, dtype=dtype, device=DEV)
    _ops().rmsnorm(x.to(DEV), w.to(DEV), out, eps)
    _close(out, P.plain_rmsnorm(x, w, eps), dtype)
    # library routine for the same formula
    lib = torch.nn.functional.rms_norm(x.double(), (d,), w.double(), eps)
    _close(out, lib, dtype)
    # gathered rows with an output scale
    rows = torch.tensor([T - 1, 0, T // 2], dtype=torch.int32)
    out2 = torch.empty(3, d, dtype=dtype, device=DEV)
    _ops().rmsnorm(x.to(DEV), w.to(DEV), out2, eps, 4.0, rows.to(DEV))
    _close(out2, P.plain_rmsnorm(x[rows.long()], w, eps) * 4.0, dtype)


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("T,d", [(3, 96), (40, 200), (9, 2304), (2050, 200), (1100, 2304), (1030, 5000)])   # the last three: many rows
def test_add_rmsnorm_and_residual_add(dtype, T, d):
    g = torch.Generator().manual_seed(3)
    x = torch.randn(T, d, generator=g)
    y = torch.randn(T, d, generator=g).to(dtype)
    w = 1 + 0.1 * torch.randn(d, generator=g)
    xd = x.to(DEV).clone()
    out = torch.empty(T, d, dtype=dtype, device=DEV)
    _ops().add_rmsnorm(xd, y.to(DEV), 0.7, w.to(DEV), out, 1e-5)
    xs = x.double() + 0.7 * y.double()
    _close(xd, xs, torch.float32)
    _close(out, P.plain_rmsnorm(xs, w, 1e-5), dtype)
    xd2 = x.to(DEV).clone()
    _ops().residual_add(xd2, y.to(DEV), 0.7)
    _close(xd2, xs, torch.float32)


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("T,di", [(1, 160), (29, 344), (7, 5760)])
def test_swiglu(dtype, T, di):
    g = torch.Generator().manual_seed(4)
    gu = (torch.randn(T, 2 * di, generator=g) * 2).to(dtype)
    out = torch.empty(T, di, dtype=dtype, device=DEV)
    _ops().swiglu(gu.to(DEV), out)
    want = P.plain_swiglu(gu[:, :di], gu[:, di:])
    _close(out, want, dtype)
    lib = torch.nn.functional.silu(gu[:, :di].double()) * gu[:, di:].double()
    _close(out, lib, dtype)
    # swapped arguments must not pass
    wrong = P.plain_swiglu(gu[:, di:], gu[:, :di])
    assert float((out.double().cpu() - wrong).abs().max()) > 0.1


# ---------------------------------------------------------------------------
def _paged(k, v, page_size, dtype, seed=0, extra_pages=3):
    """Scatter contiguous k, v [t, nkvh, dh] into shuffled pages; returns planes and the block table."""
    t, nkvh, dh = k.shape
    n_pages = (t + page_size - 1) // page_size
    g = torch.Generator().manual_seed(seed)
    perm = torch.randperm(n_pages + extra_pages, generator=g)[:n_pages]
    kc = torch.full((n_pages + extra_pages, nkvh, page_size, dh), float("nan")).to(dtype)
    vc = torch.full_like(kc, float("nan"))
    for j in range(t):
        kc[perm[j // page_size], :, j % page_size] = k[j].to(dtype)
        vc[perm[j // page_size], :, j % page_size] = v[j].to(dtype)
    return kc, vc, perm.to(torch.int32)


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("nh,nkvh,dh,rot,page", [(4, 2, 16, 16, 16), (3, 3, 32, 32, 32), (6, 2, 64, 64, 16),
                                                  (5, 1, 48, 32, 16), (2, 2, 128, 128, 64)])
def test_rope_kv_write(dtype, nh, nkvh, dh, rot, page):
    g = torch.Generator().manual_seed(5)
    T, max_pos = 23, 300
    H = (nh + 2 * nkvh) * dh
    qkv = torch.randn(T, H, generator=g).to(dtype)
    pos = torch.randint(0, max_pos, (T,), generator=g, dtype=torch.int32)
    n_pages = 6
    slots = torch.randperm(n_pages * page, generator=g)[:T].to(torch.int32)
    half = rot // 2
    sin, cos = P.plain_rope_tables(rot, 10000.0, max_pos)
    kc = torch.zeros(n_pages, nkvh, page, dh, dtype=dtype, device=DEV)
    vc = torch.zeros_like(kc)
    q_dev = qkv.to(DEV).clone()
    _ops().rope_kv_write(q_dev, pos.to(DEV), cos.float().to(DEV), sin.float().to(DEV), kc, vc, slots.to(DEV),
                         nh, nkvh, dh, rot, page)

    def rot_half(x):          # pairs (j, j + rot/2) of each head; dims beyond rot pass through
        x = x.double()
        a, b = x[..., :half], x[..., half:rot]
        c, s = cos[pos.long()][:, None, :], sin[pos.long()][:, None, :]
        return torch.cat([a * c - b * s, a * s + b * c, x[..., rot:]], dim=-1)

    heads = qkv.double().reshape(T, nh + 2 * nkvh, dh)
    want_q = rot_half(heads[:, :nh])
    want_k = rot_half(heads[:, nh:nh + nkvh])
    want_v = heads[:, nh + nkvh:]
    got = q_dev.cpu().double().reshape(T, nh + 2 * nkvh, dh)
    _close(got[:, :nh], want_q, dtype)
    kc_c, vc_c = kc.cpu().double(), vc.cpu().double()
    for t in range(T):
        pg, off = int(slots[t]) // page, int(slots[t]) % page
        _close(kc_c[pg, :, off], want_k[t], dtype, scale=float(want_k.abs().max()))
        _close(vc_c[pg, :, off], want_v[t], dtype, scale=float(want_v.abs().max()))
    if rot == dh:
        # the reference's form: adjacent pairs on row-permuted projections (scripts/jiuge.py:217-227)
        perm = P.permute_rows_to_adjacent_pairs(torch.arange(dh, dtype=torch.float64)[:, None], 1, dh)[:, 0].long()
        adj = P.plain_rope_adjacent(heads[:, :nh][..., perm], pos.tolist(), sin, cos)
        _close(got[:, :nh][..., perm], adj, dtype)


def _attention_case(dtype, nh, nkvh, dh, page, lens, window, seed, impl, table_width=0, groups=0, n_split=3, parts=None,
                    pages_given_back=False):
    """lens: list of (past, new) per request.  Returns (got, want) [T, nh*dh].  table_width pads
    the block tables with unused columns; groups is passed to the prompt-portion kernel; parts = (parts, part_len)
    cuts the prompt tiles' walks over the keys (the kernel is then launched twice: its arrival counters must come
    back to zero).  pages_given_back (with a window): the block-table entries of pages that lie wholly before the
    window of the step's first token name a page full of NaN, as if the manager had given them to someone else."""
    ops = _ops()
    g = torch.Generator().manual_seed(seed)
    scale = 1.0 / math.sqrt(dh)
    qs, want, token_req, positions, tables, kcs, vcs = [], [], [], [], [], [], []
    page_base = 0
    for r, (past, new) in enumerate(lens):
        t = past + new
        q = torch.randn(new, nh, dh, generator=g).to(dtype)
        k = torch.randn(t, nkvh, dh, generator=g).to(dtype)
        v = torch.randn(t, nkvh, dh, generator=g).to(dtype)
        want.append(P.plain_attention(q, k, v, scale, past, window).reshape(new, nh * dh))
        kc, vc, bt = _paged(k, v, page, dtype, seed=seed + r)
        if pages_given_back and window:
            gone = max(0, past - window + 1) // page
            spare = next(i for i in range(kc.shape[0]) if i not in set(bt.tolist()))      # an unused page: NaN throughout
            bt = bt.clone()
            bt[:gone] = spare
        kcs.append(kc); vcs.append(vc)
        tables.append(bt + page_base)
        page_base += kc.shape[0]
        qs.append(q.reshape(new, nh * dh))
        token_req += [r] * new
        positions += list(range(past, t))
    maxb = max(max(len(b) for b in tables), table_width)
    bt = torch.zeros(len(lens), maxb, dtype=torch.int32)
    for r, b in enumerate(tables):
        bt[r, :len(b)] = b
    q = torch.cat(qs).to(DEV)
    kc, vc = torch.cat(kcs).to(DEV), torch.cat(vcs).to(DEV)
    out = torch.zeros_like(q)
    T = q.shape[0]
    tr = torch.tensor(token_req, dtype=torch.int32, device=DEV)
    ps = torch.tensor(positions, dtype=torch.int32, device=DEV)
    btd = bt.to(DEV)
    if impl == "generic":
        ops.attention_generic(q, out, kc, vc, btd, tr, ps, nh, nkvh, dh, page, scale, window or 0)
    elif impl == "decode":
        assert all(n == 1 for _, n in lens)
        pa = torch.empty(T * nh * n_split * dh, device=DEV)
        pm = torch.empty(T * nh * n_split * 2, device=DEV)
        ops.attention_decode(q, out, kc, vc, btd, None, T, tr, ps, pa, pm, nh, nkvh, dh, page, scale,
                             window or 0, n_split)
    else:
        rows = ops.attention_prefill_tile_rows()
        tiles, row0 = [], 0
        for r, (past, new) in enumerate(lens):
            for o in range(0, new, rows):
                tiles += [r, row0 + o, min(rows, new - o), past + o]
            row0 += new
        tl = torch.tensor(tiles, dtype=torch.int32, device=DEV).view(-1, 4)
        if parts:
            scratch = torch.full((ops.attention_prefill_scratch_floats(tl.shape[0], nh, dh, parts[0]),), float("nan"), device=DEV)
            counters = torch.zeros(ops.attention_prefill_counter_ints(), dtype=torch.int32, device=DEV)
            for _ in range(2):
                out.zero_()
                ops.attention_prefill(q, out, kc, vc, btd, tl, tl.shape[0], nh, nkvh, dh, page, scale, window or 0, 1,
                                      parts=parts[0], part_len=parts[1], scratch=scratch, counters=counters)
                assert int(counters.abs().sum()) == 0          # every launch leaves its arrival counters at zero
        else:
            ops.attention_prefill(q, out, kc, vc, btd, tl, tl.shape[0], nh, nkvh, dh, page, scale, window or 0, groups)
    return out, torch.cat(want)


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("nh,nkvh,dh,page", [(4, 2, 16, 16), (3, 3, 32, 32), (5, 1, 48, 16), (6, 2, 64, 16),
                                              (2, 1, 80, 64), (8, 2, 128, 64), (2, 2, 256, 16)])
@pytest.mark.parametrize("window", [None, 37])
def test_attention_generic(dtype, nh, nkvh, dh, page, window):
    lens = [(0, 1), (0, 70), (130, 1), (64, 33), (15, 2), (257, 1)]
    got, want = _attention_case(dtype, nh, nkvh, dh, page, lens, window, 11, "generic")
    _close(got, want, dtype, factor=3)


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("nh,nkvh,dh,page", [(6, 6, 64, 16), (6, 2, 64, 64), (5, 1, 64, 32), (8, 2, 128, 16),
                                              (16, 1, 128, 64)])
@pytest.mark.parametrize("window", [None, 100])
@pytest.mark.parametrize("n_split", [1, 3])          # one split writes the result itself, more go through the second pass
def test_attention_decode(dtype, nh, nkvh, dh, page, window, n_split):
    lens = [(0, 1), (1, 1), (63, 1), (64, 1), (700, 1), (255, 1), (1031, 1)]
    got, want = _attention_case(dtype, nh, nkvh, dh, page, lens, window, 12, "decode", n_split=n_split)
    _close(got, want, dtype, factor=3)


@pytest.mark.parametrize("nh,nkvh,dh,page", [(6, 6, 64, 16), (6, 2, 64, 64), (3, 1, 64, 32), (4, 2, 128, 16),
                                              (4, 4, 128, 64)])
@pytest.mark.parametrize("window", [None, 100])
@pytest.mark.parametrize("groups", [1, 2])
def test_attention_prefill_mfma(nh, nkvh, dh, page, window, groups):
    lens = [(0, 2), (0, 129), (130, 64), (64, 33), (15, 2), (257, 300), (5, 128)]
    got, want = _attention_case(torch.bfloat16, nh, nkvh, dh, page, lens, window, 13, "prefill", groups=groups)
    _close(got, want, torch.bfloat16, factor=3)


@pytest.mark.parametrize("impl,dtype,groups,parts", [("prefill", torch.bfloat16, 1, None), ("prefill", torch.bfloat16, 2, None),
                                                      ("prefill", torch.bfloat16, 1, (3, 1)), ("prefill", torch.float32, 0, None),
                                                      ("generic", torch.bfloat16, 0, None), ("generic", torch.float32, 0, None)])
@pytest.mark.parametrize("nh,nkvh,dh,page", [(6, 2, 64, 16), (3, 3, 64, 64), (4, 1, 128, 32), (2, 2, 128, 128)])
def test_attention_never_reads_pages_that_the_window_has_passed(impl, dtype, groups, parts, nh, nkvh, dh, page):
    """The cache manager gives a page back as soon as a window has passed it, and someone else may write it: the
    block-table entries before the window then name a page of NaN here, the rows of the last page beyond the last
    key are NaN anyway, and nothing of either may reach the result (a NaN value times a probability of 0 is NaN)."""
    lens = [(700, 140), (257, 300), (130, 64), (1000, 33), (90, 2), (5, 128)]
    got, want = _attention_case(dtype, nh, nkvh, dh, page, lens, 100, 43, impl, groups=groups, parts=parts, pages_given_back=True)
    assert bool(torch.isfinite(got.float()).all())
    _close(got, want, dtype, factor=3)


def test_attention_of_single_tokens_never_reads_pages_that_the_window_has_passed():
    for dtype, nh, nkvh, dh, page, n_split in [(torch.bfloat16, 6, 6, 64, 16, 1), (torch.bfloat16, 8, 2, 128, 64, 3),
                                                (torch.float32, 4, 2, 64, 32, 3), (torch.bfloat16, 16, 1, 64, 16, 2)]:
        lens = [(700, 1), (99, 1), (100, 1), (1031, 1), (163, 1)]
        got, want = _attention_case(dtype, nh, nkvh, dh, page, lens, 100, 44, "decode", n_split=n_split, pages_given_back=True)
        assert bool(torch.isfinite(got.float()).all())
        _close(got, want, dtype, factor=3)


@pytest.mark.parametrize("nh,nkvh,dh,page", [(6, 6, 64, 16), (6, 2, 64, 64), (3, 1, 64, 32), (4, 2, 128, 16), (4, 4, 128, 64)])
@pytest.mark.parametrize("window", [None, 100])
def test_attention_prefill_in_true_float32(nh, nkvh, dh, page, window):
    """Prompt portions in float32 on the matrix cores (float32 operands and accumulation): whole prompts, portions after a
    past, tiles that end inside a page, two tokens, a window; to float32 accuracy against the plain attention."""
    lens = [(0, 2), (0, 129), (130, 64), (64, 33), (15, 2), (257, 300), (5, 128), (700, 140)]
    got, want = _attention_case(torch.float32, nh, nkvh, dh, page, lens, window, 33, "prefill")
    _close(got, want, torch.float32, factor=3)


@pytest.mark.parametrize("nh,nkvh,dh,page", [(6, 6, 64, 16), (6, 2, 64, 64), (3, 1, 64, 32), (4, 2, 128, 16), (4, 4, 128, 64)])
@pytest.mark.parametrize("window", [None, 300])
@pytest.mark.parametrize("parts", [(2, 1), (3, 2), (4, 1), (8, 3)])
def test_attention_prefill_with_the_walk_over_the_keys_cut_into_parts(nh, nkvh, dh, page, window, parts):
    """Blocks of their own walk parts of a query tile's keys and the last one to arrive merges them: tiles with fewer
    key tiles than parts, tiles that start inside a page, a request of two tokens, two launches in a row."""
    lens = [(0, 2), (0, 129), (130, 64), (700, 140), (257, 300), (5, 128), (1000, 33)]
    got, want = _attention_case(torch.bfloat16, nh, nkvh, dh, page, lens, window, 23, "prefill", parts=parts)
    _close(got, want, torch.bfloat16, factor=3)


def test_attention_prefill_parts_rule_and_its_refusals():
    ops = _ops()
    assert ops.attention_prefill_parts(16, 36, 64, 2048, 256) == (2, 16)         # the benchmark's prompt: 576 blocks of 32 key tiles
    assert ops.attention_prefill_parts(4, 36, 64, 2048, 256) == (3, 11)          # a portion of 512 after 1,536: few blocks, three parts
    assert ops.attention_prefill_parts(4, 24, 64, 1024, 256) == (3, 6)           # few blocks: walks of 12 key tiles and more are cut
    assert ops.attention_prefill_parts(2, 24, 64, 1280, 256) == (4, 5)           # very few blocks and 20 key tiles: four parts
    assert ops.attention_prefill_parts(4, 24, 64, 704, 256)[0] == 1              # 11 key tiles: left whole
    assert ops.attention_prefill_parts(4, 32, 128, 1024, 256) == (2, 8) and ops.attention_prefill_parts(2, 32, 128, 1280, 256) == (4, 5)
    assert ops.attention_prefill_parts(8, 32, 128, 1024, 256)[0] == 1            # a block a unit at head size 128: two wave groups do it
    assert ops.attention_prefill_parts(4, 36, 64, 1024, 256)[0] == 1             # short walks are left whole
    assert ops.attention_prefill_parts(32, 36, 64, 4096, 256)[0] == 1            # many blocks too
    assert ops.attention_prefill_parts(16, 32, 128, 2048, 256)[0] == 1 and ops.attention_prefill_parts(4, 40, 128, 4096, 256)[0] == 3
    assert ops.attention_prefill_scratch_floats(4, 36, 64, 4) == 4 * 36 * 4 * 256 * 34
    q = torch.zeros(128, 64, dtype=torch.bfloat16, device=DEV)
    kc = torch.zeros(2, 1, 64, 64, dtype=torch.bfloat16, device=DEV)
    bt = torch.zeros(1, 2, dtype=torch.int32, device=DEV)
    tl = torch.tensor([[0, 0, 128, 0]], dtype=torch.int32, device=DEV)
    small = torch.zeros(16, device=DEV)
    counters = torch.zeros(ops.attention_prefill_counter_ints(), dtype=torch.int32, device=DEV)
    with pytest.raises(ops.KernelError):        # scratch memory too small for two parts
        ops.attention_prefill(q, torch.zeros_like(q), kc, kc, bt, tl, 1, 1, 1, 64, 64, 0.125, 0, 1, parts=2, part_len=1, scratch=small,
                              counters=counters)
    with pytest.raises(ops.KernelError):        # parts go with one wave group only
        ops.attention_prefill(q, torch.zeros_like(q), kc, kc, bt, tl, 1, 1, 1, 64, 64, 0.125, 0, 2, parts=2, part_len=1,
                              scratch=torch.zeros(2 * 256 * 34, device=DEV), counters=counters)
    with pytest.raises(ops.KernelError):        # a cut walk without arrival counters of the caller's
        ops.attention_prefill(q, torch.zeros_like(q), kc, kc, bt, tl, 1, 1, 1, 64, 64, 0.125, 0, 1, parts=2, part_len=1,
                              scratch=torch.zeros(2 * 256 * 34, device=DEV))


@pytest.mark.parametrize("impl,dtype,nh,nkvh,dh", [("decode", torch.bfloat16, 6, 6, 64), ("decode", torch.float32, 4, 4, 128),
                                                     ("decode", torch.bfloat16, 6, 2, 64), ("decode", torch.float32, 6, 2, 64),
                                                     ("decode", torch.bfloat16, 16, 1, 128),
                                                     ("prefill1", torch.bfloat16, 6, 2, 64), ("prefill2", torch.bfloat16, 6, 2, 64),
                                                     ("prefill1", torch.bfloat16, 4, 4, 128), ("prefill2", torch.bfloat16, 4, 2, 128)])
def test_attention_with_block_tables_too_wide_to_stage(impl, dtype, nh, nkvh, dh):
    """Block tables wider than the page-id staging area: the kernels read page ids from memory."""
    if impl == "decode":
        lens = [(0, 1), (63, 1), (700, 1), (255, 1)]
        got, want = _attention_case(dtype, nh, nkvh, dh, 16, lens, 100 if nh == 6 else None, 15, "decode", table_width=2100)
    else:
        lens = [(0, 129), (130, 64), (257, 300)]
        got, want = _attention_case(dtype, nh, nkvh, dh, 16, lens, None, 16, "prefill", table_width=2100,
                                    groups=int(impl[-1]))
    _close(got, want, dtype, factor=3)


def test_attention_special_cases():
    """One key: the output is that value row.  Equal scores: the mean of the values.
    No rotation, no mask (the last row of a prompt): the library's attention."""
    dtype, nh, nkvh, dh, page = torch.float32, 2, 2, 32, 16
    ops = _ops()
    g = torch.Generator().manual_seed(14)
    t = 40
    k = torch.randn(t, nkvh, dh, generator=g)
    v = torch.randn(t, nkvh, dh, generator=g)
    q = torch.randn(t, nh, dh, generator=g)
    kc, vc, bt = _paged(k, v, page, dtype)
    tr = torch.zeros(t, dtype=torch.int32, device=DEV)
    ps = torch.arange(t, dtype=torch.int32, device=DEV)
    out = torch.empty(t, nh * dh, device=DEV)
    scale = 1 / math.sqrt(dh)
    ops.attention_generic(q.reshape(t, -1).to(DEV), out, kc.to(DEV), vc.to(DEV), bt[None].to(DEV), tr, ps,
                          nh, nkvh, dh, page, scale, 0)
    out = out.cpu().reshape(t, nh, dh)
    _close(out[0], v[0], dtype)                                   # position 0 sees one key
    lib = torch.nn.functional.scaled_dot_product_attention(
        q.double().transpose(0, 1), k.double().transpose(0, 1), v.double().transpose(0, 1), is_causal=True)
    _close(out, lib.transpose(0, 1), dtype, factor=5)
    # equal scores: q = 0
    out0 = torch.empty(t, nh * dh, device=DEV)
    ops.attention_generic(torch.zeros(t, nh * dh, device=DEV), out0, kc.to(DEV), vc.to(DEV), bt[None].to(DEV),
                          tr, ps, nh, nkvh, dh, page, scale, 0)
    _close(out0.cpu().reshape(t, nh, dh)[-1], v.double().mean(0), dtype, factor=5)


@pytest.mark.parametrize("impl,dtype", [("generic", torch.float32), ("generic", torch.bfloat16),
                                        ("decode", torch.float32), ("decode", torch.bfloat16),
                                        ("prefill", torch.bfloat16), ("prefill", torch.float32)])
def test_attention_far_key_and_window_edge(impl, dtype):
    """One far key among hundreds is made to stand out (its score dwarfs the rest):
    the output must be its value row.  With a window, the key at its edge counts
    and the key one step beyond does not."""
    ops = _ops()
    nh = nkvh = 2
    dh, page = 64, 16
    g = torch.Generator().manual_seed(15)
    t = 777
    past = t - 1 if impl != "prefill" else t - 150
    new = t - past
    scale = 1 / math.sqrt(dh)
    for window, far, inside in [(None, 3, True), (None, 401, True), (300, t - 300, True), (300, t - 301, False)]:
        k = torch.randn(t, nkvh, dh, generator=g) * 0.1
        v = torch.randn(t, nkvh, dh, generator=g)
        q = torch.randn(new, nh, dh, generator=g) * 0.1
        k[far, :, 7] = 40.0
        q[-1, :, 7] = 40.0            # the last query's score against key `far` is 1600/8 = 200
        kc, vc, bt = _paged(k.to(dtype), v.to(dtype), page, dtype, seed=far)
        kc, vc = kc.to(DEV), vc.to(DEV)
        qd = q.to(dtype).reshape(new, -1).to(DEV)
        out = torch.zeros(new, nh * dh, dtype=dtype, device=DEV)
        tr = torch.zeros(new, dtype=torch.int32, device=DEV)
        ps = torch.arange(past, t, dtype=torch.int32, device=DEV)
        btd = bt[None].contiguous().to(DEV)
        if impl == "generic":
            ops.attention_generic(qd, out, kc, vc, btd, tr, ps, nh, nkvh, dh, page, scale, window or 0)
        elif impl == "decode":
            pa = torch.empty(nh * 4 * dh, device=DEV); pm = torch.empty(nh * 4 * 2, device=DEV)
            ops.attention_decode(qd, out, kc, vc, btd, None, 1, tr, ps, pa, pm, nh, nkvh, dh, page, scale,
                                 window or 0, 4)
        else:
            rows = ops.attention_prefill_tile_rows()
            tiles = []
            for o in range(0, new, rows):
                tiles += [0, o, min(rows, new - o), past + o]
            tl = torch.tensor(tiles, dtype=torch.int32, device=DEV).view(-1, 4)
            ops.attention_prefill(qd, out, kc, vc, btd, tl, tl.shape[0], nh, nkvh, dh, page, scale, window or 0)
        last = out[-1].float().cpu().reshape(nh, dh)
        vfar = v[far].to(dtype).float()
        hit = float((last - vfar).abs().max()) < 0.05
        assert hit == inside, "window %s, key %d: expected %s" % (window, far, "seen" if inside else "not seen")


# ---------------------------------------------------------------------------
@pytest.mark.parametrize("cdtype", DT)
@pytest.mark.parametrize("M,N,K", [(1, 331, 200), (8, 2304, 2304), (16, 509, 96), (17, 1000, 344), (64, 777, 5760),
                                   (3, 122753, 64), (130, 300, 100),
                                   # 32,768 weight rows and more with up to 16 rows: waves own whole weight tiles;
                                   # 8 waves a block, 16 where the token rows take most of the LDS, few groups of K
                                   (7, 50007, 2304), (16, 35001, 1032), (13, 40000, 4104), (1, 33000, 8)])
def test_gemm_nt(cdtype, M, N, K):
    g = torch.Generator().manual_seed(16)
    a = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w = torch.randn(N, K, generator=g).to(torch.bfloat16)
    out = torch.empty(M, N, dtype=cdtype, device=DEV)
    _ops().gemm_nt(a.to(DEV), w.to(DEV), out, 0.5)
    want = 0.5 * P.plain_linear(a, w)
    _close(out, want, cdtype, factor=2)


@pytest.mark.parametrize("dtype,cdtype", [(torch.bfloat16, torch.bfloat16), (torch.bfloat16, torch.float32),
                                          (torch.float32, torch.float32)])
@pytest.mark.parametrize("M,N,K", [(40, 331, 200), (300, 1000, 344)])
def test_library_product_before_and_after_timing_its_algorithms(dtype, cdtype, M, N, K):
    """The library product called directly: with the library's first choice, and again after every
    algorithm was timed (with a buffer overwritten between the launches) and the fastest kept."""
    ops = _ops()
    g = torch.Generator().manual_seed(21)
    a = torch.randn(M, K, generator=g).to(dtype)
    w = torch.randn(N, K, generator=g).to(dtype)
    want = 0.25 * P.plain_linear(a, w)
    ad, wd = a.to(DEV), w.to(DEV)
    out = torch.full((M, N), float("nan"), dtype=cdtype, device=DEV)
    ops.matmul_library(ad, wd, out, 0.25)
    _close(out, want, cdtype if dtype == torch.bfloat16 else torch.float32, factor=2)
    flush = torch.empty(8 << 20, dtype=torch.uint8, device=DEV)
    assert ops.matmul_library_tune(ad, wd, out, reps=2, flush=flush) >= 1
    out.fill_(float("nan"))
    ops.matmul_library(ad, wd, out, 0.25)
    _close(out, want, cdtype if dtype == torch.bfloat16 else torch.float32, factor=2)
    # a row count near the timed one, first seen now, may take over the timed algorithm
    for rows in (M - M // 10, M - 1):
        part = torch.full((rows, N), float("nan"), dtype=cdtype, device=DEV)
        ops.matmul_library(ad[:rows], wd, part, 0.25)
        _close(part, want[:rows], cdtype if dtype == torch.bfloat16 else torch.float32, factor=2)


def test_library_float32_product_is_true_float32():
    """The float32 path's matrix products must not run in a reduced-precision mode."""
    from infinicore_infer_amd.parts.linear import linear
    g = torch.Generator().manual_seed(17)
    a = torch.randn(200, 2304, generator=g)
    w = torch.randn(500, 2304, generator=g)
    out = torch.empty(200, 500, device=DEV)
    linear(a.to(DEV), w.to(DEV), out)
    want = a.double() @ w.double().t()
    err = float((out.cpu().double() - want).abs().max()) / float(want.abs().max())
    assert err < 5e-6, "float32 product error %.3g: a reduced-precision mode is on" % err


# ---------------------------------------------------------------------------
@pytest.mark.parametrize("V", [256, 509, 122753, 300001])     # the last: beyond what the per-run masses cover
def test_sampling(V):
    ops = _ops()
    g = torch.Generator().manual_seed(18)
    cases = [(0.0, 0, 1.0), (1.0, 1, 1.0), (1.0, 0, 1.0), (0.7, 5, 1.0), (1.3, 0, 0.8), (0.9, 40, 0.6),
             (2.0, V, 0.95), (1.0, 3, 0.01)]
    R = len(cases) * 6
    logits = torch.randn(R, V, generator=g) * 3
    logits[0, 10] = logits[0, 20] = 50.0                  # equal maxima: the lowest index wins
    temps = torch.tensor([c[0] for c in cases] * 6)
    ks = torch.tensor([c[1] for c in cases] * 6, dtype=torch.int32)
    ps = torch.tensor([c[2] for c in cases] * 6)
    us = torch.rand(R, generator=g)
    out = torch.empty(R, dtype=torch.int32, device=DEV)
    ops.sample(logits.to(DEV), out, temps.to(DEV), ks.to(DEV), ps.to(DEV), us.to(DEV))
    got = out.cpu().tolist()
    assert got[0] == 10
    for r in range(R):
        want = P.plain_sample(logits[r], float(temps[r]), int(ks[r]), float(ps[r]), float(us[r]))
        assert got[r] == want, "row %d (T=%g k=%d p=%g u=%g): got %d, plain %d" % (
            r, temps[r], ks[r], ps[r], us[r], got[r], want)
    # argmax for every row when no temperature is given, in one kernel and in two stages
    want = [int(torch.argmax(logits[r])) for r in range(R)]
    want[0] = 10
    ops.sample(logits.to(DEV), out)
    assert out.cpu().tolist() == want
    out.zero_()
    ops.argmax(logits.to(DEV), out, torch.empty(64 * R, device=DEV), torch.empty(64 * R, dtype=torch.int32, device=DEV))
    assert out.cpu().tolist() == want


@pytest.mark.parametrize("V", [5003, 122753])
def test_sampling_where_the_short_list_does_not_apply_or_ties_cross_its_edge(V):
    """Rows made so that the kernel's ways through a row all occur: ties across the k-th place (kept
    together), a k so large and a distribution so flat that the candidates do not fit in LDS, all logits
    equal, all negative, a draw at either end."""
    ops = _ops()
    g = torch.Generator().manual_seed(23)
    rows, params = [], []

    def add(row, t, k, p, u):
        rows.append(row)
        params.append((t, k, p, u))

    base = torch.randn(V, generator=g) * 3
    tied = base.clone()
    top = torch.topk(tied, 12).indices
    tied[top[4:]] = float(tied[top[4]])                         # places 5..12 share one value
    for k in (5, 6, 12, 13):
        add(tied, 1.0, k, 1.0, 0.999)
        add(tied, 0.8, k, 0.7, 0.5)
    add(base, 1.0, V - 1, 1.0, 0.37)                            # top-k cuts one token: no short list
    add(base, 1.5, V // 3, 0.9, 0.61)
    add(base * 0.01, 1.0, 0, 0.9, 0.42)                         # nearly flat: top-p keeps most of the row
    add(torch.full((V,), 1.25), 1.0, 7, 0.5, 0.73)              # all equal: everything stays together
    add(-10.0 - torch.rand(V, generator=g), 0.9, 40, 0.8, 0.2)  # all negative
    add(base, 1.0, 50, 0.9, 0.0)                                # the draw's ends
    add(base, 1.0, 50, 0.9, 1.0)
    add(base, 1.0, 0, 1.0, 0.0)
    add(base, 1.0, 0, 1.0, 1.0)
    add(base, 0.05, 0, 0.999, 0.5)                              # a cold temperature: most masses round to zero
    logits = torch.stack(rows)
    R = len(rows)
    col = lambda j, dt: torch.tensor([q[j] for q in params], dtype=dt).to(DEV)
    out = torch.empty(R, dtype=torch.int32, device=DEV)
    ops.sample(logits.to(DEV), out, col(0, torch.float32), col(1, torch.int32), col(2, torch.float32), col(3, torch.float32))
    got = out.cpu().tolist()
    for r, (t, k, p, u) in enumerate(params):
        want = P.plain_sample(logits[r], t, k, p, float(torch.tensor(u, dtype=torch.float32)))
        assert got[r] == want, "row %d (T=%g k=%d p=%g u=%g): got %d, plain %d" % (r, t, k, p, u, got[r], want)


def test_sampling_distribution():
    """Many draws at temperature 1 follow softmax (chi-square against torch.softmax)."""
    ops = _ops()
    g = torch.Generator().manual_seed(19)
    V, n = 12, 20000
    row = torch.randn(V, generator=g)
    logits = row[None].expand(n, V).contiguous().to(DEV)
    us = torch.rand(n, generator=g).to(DEV)
    out = torch.empty(n, dtype=torch.int32, device=DEV)
    ops.sample(logits, out, torch.ones(n, device=DEV), torch.zeros(n, dtype=torch.int32, device=DEV),
               torch.ones(n, device=DEV), us)
    counts = torch.bincount(out.cpu().long(), minlength=V).double()
    expect = torch.softmax(row.double(), 0) * n
    chi2 = float(((counts - expect) ** 2 / expect).sum())
    assert chi2 < 40.0, "chi-square %.1f over %d bins" % (chi2, V)       # 11 dof: p(chi2 > 40) < 1e-4


@pytest.mark.parametrize("cdtype", DT)
@pytest.mark.parametrize("M,di,K", [(1, 344, 200), (8, 5760, 2304), (16, 256, 96), (5, 130, 100), (3, 3840, 1536),
                                    (5, 8400, 136), (2, 8400, 2048),     # the last two: more tiles than one round of blocks takes
                                    (17, 5760, 2304), (32, 3840, 1536), (25, 344, 192), (31, 16384, 128)])   # 17..32 rows: two row tiles
def test_gemm_nt_with_swiglu_output(cdtype, M, di, K):
    """The gate/up projection with the activation in its epilogue equals the plain product
    followed by the SwiGLU kernel."""
    g = torch.Generator().manual_seed(21)
    h = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w = (torch.randn(2 * di, K, generator=g) * 0.1).to(torch.bfloat16)
    out = torch.empty(M, di, dtype=cdtype, device=DEV)
    if M > 16 and cdtype != torch.bfloat16:          # two row tiles exist for bfloat16 results only: refused, not computed wrongly
        with pytest.raises(_ops().KernelError):
            _ops().gemm_nt(h.to(DEV), w.to(DEV), out, swiglu_output=True)
        return
    assert M <= _ops().gemm_epilogue_rows("swiglu", h, w)
    _ops().gemm_nt(h.to(DEV), w.to(DEV), out, swiglu_output=True)
    rnd = P.round_bf16 if cdtype == torch.bfloat16 else (lambda t: t)
    gu = rnd(P.plain_linear(h, w))
    _close(out, P.plain_swiglu(gu[:, :di], gu[:, di:]), cdtype, factor=2 if cdtype == torch.bfloat16 else 50)


@pytest.mark.parametrize("M,nh,nkvh,dh,K,page", [(1, 4, 2, 32, 96, 16), (8, 6, 2, 64, 200, 16), (16, 3, 3, 64, 2304, 64),
                                                 (5, 4, 1, 128, 344, 32), (3, 36, 36, 64, 2304, 64),
                                                 # 17..32 rows: two row tiles per block (whole-line weight loads)
                                                 (17, 6, 2, 64, 1536, 64), (32, 3, 3, 64, 2304, 16), (25, 4, 1, 128, 640, 32),
                                                 (20, 5, 5, 32, 192, 16), (31, 36, 36, 64, 2304, 64)])
@pytest.mark.parametrize("tile_rows", [0, 16, 8, 4])
def test_gemm_qkv_rope(M, nh, nkvh, dh, K, page, tile_rows):
    """The fused projection + rotary + cache write equals the plain product followed by the
    rotary/cache-write kernel, with every number of used rows per tile (0: chosen from the heads)."""
    g = torch.Generator().manual_seed(31)
    ops = _ops()
    H = (nh + 2 * nkvh) * dh
    h = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w = (torch.randn(H, K, generator=g) * 0.1).to(torch.bfloat16)
    max_pos, n_pages = 300, 5
    pos = torch.randint(0, max_pos, (M,), generator=g, dtype=torch.int32)
    slots = torch.randperm(n_pages * page, generator=g)[:M].to(torch.int32)
    if M > 2:
        slots[1] = -1                        # a row without a cache slot writes nothing
    sin, cos = P.plain_rope_tables(dh, 10000.0, max_pos)
    sin, cos = sin.float().to(DEV), cos.float().to(DEV)
    kc = torch.zeros(n_pages, nkvh, page, dh, dtype=torch.bfloat16, device=DEV)
    vc = torch.zeros_like(kc)
    qkv = torch.zeros(M, H, dtype=torch.bfloat16, device=DEV)
    ops.gemm_qkv_rope(h.to(DEV), w.to(DEV), qkv, pos.to(DEV), slots.to(DEV), cos, sin, kc, vc, nh, nkvh, dh, page,
                      tile_rows=tile_rows)
    # the two-kernel path
    kc2, vc2 = torch.zeros_like(kc), torch.zeros_like(vc)
    ref = torch.empty(M, H, dtype=torch.bfloat16, device=DEV)
    ops.gemm_nt(h.to(DEV), w.to(DEV), ref)
    ops.rope_kv_write(ref, pos.to(DEV), cos, sin, kc2, vc2, slots.to(DEV), nh, nkvh, dh, dh, page)
    _close(qkv[:, :nh * dh], ref[:, :nh * dh], torch.bfloat16)
    _close(kc, kc2, torch.bfloat16)
    _close(vc, vc2, torch.bfloat16)
    assert float(kc2.abs().max()) > 0 and float(vc2.abs().max()) > 0


@pytest.mark.parametrize("M,N,K,N2", [(1, 200, 344, 331), (8, 2304, 2304, 6912), (16, 96, 509, 64), (5, 4096, 130, 50),
                                      (3, 1536, 3840, 1000), (7, 304, 8264, 130), (16, 512, 16384, 96),
                                      (5, 200, 344, 33331), (16, 1000, 72, 40002)])
def test_norm_split_over_two_products(M, N, K, N2):
    """Residual add + RMS norm between two products, split over them: the first product's
    epilogue adds to the stream and stores x * w with sums of squares; the second applies the
    row factors to its result.  Equals product, add, norm, product done one after the other."""
    g = torch.Generator().manual_seed(41)
    ops = _ops()
    a = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w1 = (torch.randn(N, K, generator=g) * 0.1).to(torch.bfloat16)
    w2 = (torch.randn(N2, N, generator=g) * 0.1).to(torch.bfloat16)
    x = torch.randn(M, N, generator=g) * 3.0
    gw = torch.rand(N, generator=g) + 0.5
    beta, eps, alpha2 = 0.37, 1e-5, 0.7
    xd = x.to(DEV)
    y = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
    sumsq = torch.full((ops.residual_parts(N), 16), float("nan"), device=DEV)
    ops.gemm_nt(a.to(DEV), w1.to(DEV), y, residual=(xd, gw.to(DEV), beta, sumsq))
    # the stream after the add: the product is rounded to bfloat16 before it is added, so the stream
    # may differ from the exact sum by that rounding (relative to the product), no more
    delta = P.plain_linear(a, w1)
    _close(xd, x.double() + beta * delta, torch.bfloat16, scale=beta * float(delta.abs().max()))
    assert float((xd.cpu() - x).abs().max()) > 0
    # the half-done rows and the sums follow from the stream as it now is
    x_new = xd.double().cpu()
    _close(y, x_new * gw.double(), torch.bfloat16)
    ss = sumsq.double().cpu()
    assert torch.isfinite(ss).all()
    assert float(ss[:, M:].abs().max()) == 0.0 if M < 16 else True      # rows that do not exist add nothing
    _close(ss.sum(0)[:M], (x_new * x_new).sum(1), torch.float32, factor=10)
    # second product with the row factors, float32 and bfloat16 results
    for cdtype in DT:
        out = torch.empty(M, N2, dtype=cdtype, device=DEV)
        ops.gemm_nt(y, w2.to(DEV), out, alpha=alpha2, row_factor=(sumsq, N, eps))
        rs = torch.rsqrt((x_new * x_new).mean(1, keepdim=True) + eps)
        want = alpha2 * rs * P.plain_linear(y.cpu(), w2)
        _close(out, want, cdtype, factor=1 if cdtype == torch.bfloat16 else 100)
        # and it is the norm: compare with norm-then-product in float64 (bf16 rounding of the rows apart)
        full = alpha2 * P.plain_linear(P.plain_rmsnorm(x_new, gw, eps), w2)
        _close(out, full, torch.bfloat16, factor=2)
    # the activation and the rotary epilogues take the factors too
    if N2 % 2 == 0:
        act = torch.empty(M, N2 // 2, dtype=torch.bfloat16, device=DEV)
        ops.gemm_nt(y, w2.to(DEV), act, swiglu_output=True, row_factor=(sumsq, N, eps))
        gu = P.round_bf16(rs * P.plain_linear(y.cpu(), w2))
        _close(act, P.plain_swiglu(gu[:, :N2 // 2], gu[:, N2 // 2:]), torch.bfloat16, factor=2)


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("M,N,K", [(1, 33001, 2048), (7, 40000, 2112), (16, 32771, 2304)])
def test_the_head_product_with_whole_line_weight_loads(M, N, K, out_dtype):
    """Very many weight rows (the output head): from rows of 4 KB that are whole cache lines the kernel whose waves own
    whole weight tiles reads them line by line through LDS; switched off it loads in operand layout.  The two add the same
    products in the same order, so they agree to the bit, and both give the plain product."""
    ops = _ops()
    g = torch.Generator().manual_seed(67)
    a = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w = (torch.randn(N, K, generator=g) * 0.1).to(torch.bfloat16)
    ad, wd = a.to(DEV), w.to(DEV)
    got = {}
    for on in (1, 0):
        out = torch.full((M, N), float("nan"), dtype=out_dtype, device=DEV)
        ops.gemm_nt(ad, wd, out, 0.25, whole_lines=bool(on))
        got[on] = out.cpu()
    assert torch.equal(got[1], got[0])
    _close(got[1], 0.25 * P.plain_linear(a, w), out_dtype, factor=20 if out_dtype == torch.float32 else 2)


@pytest.mark.parametrize("M", [1, 3, 8, 16])
@pytest.mark.parametrize("N,K", [(331, 192), (2304, 2304), (1000, 1536), (512, 8192 + 64), (12000, 640)])
def test_whole_line_weight_loads_equal_loads_in_operand_layout(M, N, K):
    """With K a multiple of 64 the few-row products read their weights in whole cache lines and pass them through LDS;
    switched off, the same entry points load in operand layout.  Both must give the plain product, the activation
    epilogue and the residual epilogue alike (rows of 16 KB and more: a wave owns a run of k-steps)."""
    ops = _ops()
    g = torch.Generator().manual_seed(61)
    a = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w = (torch.randn(N, K, generator=g) * 0.1).to(torch.bfloat16)
    x = torch.randn(M, N, generator=g)
    gw = torch.rand(N, generator=g) + 0.5
    ad, wd = a.to(DEV), w.to(DEV)
    got = {}
    for on in (1, 0):
        lines = bool(on)
        plain = torch.empty(M, N, dtype=torch.float32, device=DEV)
        ops.gemm_nt(ad, wd, plain, 0.5, whole_lines=lines)
        res = None
        if N % 2 == 0:
            act = torch.empty(M, N // 2, dtype=torch.bfloat16, device=DEV)
            ops.gemm_nt(ad, wd, act, swiglu_output=True, whole_lines=lines)
            xd = x.to(DEV)
            y = torch.zeros(M, N, dtype=torch.bfloat16, device=DEV)
            if ops.residual_parts(N) <= ops.max_sumsq_parts():
                sumsq = torch.zeros(ops.residual_parts(N), 16, device=DEV)
                ops.gemm_nt(ad, wd, y, residual=(xd, gw.to(DEV), 0.3, sumsq), whole_lines=lines)
            res = (act.float().cpu(), xd.cpu(), y.float().cpu())
        got[on] = (plain.cpu(), res)
    want = 0.5 * P.plain_linear(a, w)
    for on in (1, 0):
        _close(got[on][0], want, torch.float32, factor=20)
    if got[1][1] is not None:
        gu = P.round_bf16(P.plain_linear(a, w))
        for on in (1, 0):
            act, xs, y = got[on][1]
            _close(act, P.plain_swiglu(gu[:, :N // 2], gu[:, N // 2:]), torch.bfloat16, factor=2)
            if ops.residual_parts(N) <= ops.max_sumsq_parts():
                _close(xs, x.double() + 0.3 * gu, torch.bfloat16, scale=0.3 * float(gu.abs().max()))
                _close(y, xs.double() * gw.double(), torch.bfloat16)


def test_gemm_qkv_rope_with_row_factors():
    g = torch.Generator().manual_seed(43)
    ops = _ops()
    M, nh, nkvh, dh, K, page = 7, 6, 2, 64, 200, 16
    H = (nh + 2 * nkvh) * dh
    yv = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w = (torch.randn(H, K, generator=g) * 0.1).to(torch.bfloat16)
    sumsq = (torch.rand(ops.residual_parts(K), 16, generator=g) * 4.0).to(DEV)
    eps = 1e-6
    rs = torch.rsqrt(sumsq.double().cpu().sum(0)[:M, None] / K + eps)
    pos = torch.randint(0, 300, (M,), generator=g, dtype=torch.int32)
    slots = torch.randperm(5 * page, generator=g)[:M].to(torch.int32)
    sin, cos = P.plain_rope_tables(dh, 10000.0, 300)
    sin, cos = sin.float().to(DEV), cos.float().to(DEV)
    kc = torch.zeros(5, nkvh, page, dh, dtype=torch.bfloat16, device=DEV)
    vc = torch.zeros_like(kc)
    qkv = torch.zeros(M, H, dtype=torch.bfloat16, device=DEV)
    ops.gemm_qkv_rope(yv.to(DEV), w.to(DEV), qkv, pos.to(DEV), slots.to(DEV), cos, sin, kc, vc, nh, nkvh, dh, page,
                      row_factor=(sumsq, K, eps))
    ref = P.round_bf16(rs * P.plain_linear(yv, w)).to(torch.bfloat16).to(DEV)
    kc2, vc2 = torch.zeros_like(kc), torch.zeros_like(vc)
    ops.rope_kv_write(ref, pos.to(DEV), cos, sin, kc2, vc2, slots.to(DEV), nh, nkvh, dh, dh, page)
    _close(qkv[:, :nh * dh], ref[:, :nh * dh], torch.bfloat16)
    _close(kc, kc2, torch.bfloat16)
    _close(vc, vc2, torch.bfloat16)


# ---------------------------------------------------------------------------
@pytest.mark.parametrize("M,N,K,S", [(1, 64, 128, 1), (17, 2304, 2304, 0), (33, 200, 344, 1), (64, 2304, 5760, 0), (48, 1000, 1096, 2),
                                      (64, 331, 64, 1), (5, 77, 72, 1), (20, 4096, 8192, 0), (64, 136, 520, 1), (31, 777, 1160, 3)])
def test_gemm_in_slices_and_the_add_norm_that_sums_them(M, N, K, S):
    """The product of 1..64 rows as float32 slices over K (sizes that are no multiple of the block's 64 columns
    or of its chunk of 128 k; slices of unequal length), against float64; then the kernel that sums the slices,
    rounds to bfloat16, adds to the residual stream and applies the norm, against the same steps in float64."""
    ops = _ops()
    g = torch.Generator().manual_seed(M * 1000 + N + K)
    a = torch.randn(M, K, generator=g).to(torch.bfloat16).to(DEV)
    w = (torch.randn(N, K, generator=g) / math.sqrt(K)).to(torch.bfloat16).to(DEV)
    assert ops.gemm_splitk_supported(a, w)
    # rows shorter than 64 elements are refused (a clamped load of the last chunk would read past the row's end)
    assert not ops.gemm_splitk_supported(a[:, :8].contiguous(), w[:, :8].contiguous())
    assert not ops.gemm_splitk_supported(a[:, :56].contiguous(), w[:, :56].contiguous())
    slices = S or ops.gemm_splitk_slices(N, K)
    parts = torch.full((slices * M * N + 64,), float("nan"), device=DEV)
    p = ops.gemm_splitk(a, w, parts, slices)
    assert p.shape == (slices, M, N)
    assert bool(torch.isnan(parts[slices * M * N:]).all())            # nothing written beyond the slices
    want = a.double().cpu() @ w.double().cpu().t()
    _close(p.double().sum(0), want, torch.float32, factor=4)
    if S == 0:                                                        # the library's own choice: slices it says are not empty
        assert 1 <= slices <= 64
    if N % 4:
        return
    x = torch.randn(M, N, generator=g).to(DEV)
    weight = (1 + 0.1 * torch.randn(N, generator=g)).to(DEV)
    out = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
    x_before = x.double().cpu()
    ops.splitk_add_rmsnorm(p, x, 0.37, weight, out, 1e-5)
    t = p[0].cpu().clone()                                            # the slices summed in float32 in the kernel's order, so
    for i in range(1, slices):                                        # that the rounding to bfloat16 (the product as it would
        t += p[i].cpu()                                               # be stored) falls the same way
    y = t.to(torch.bfloat16).double()
    x_want = x_before + 0.37 * y
    _close(x, x_want, torch.float32, factor=4)
    _close(out, P.plain_rmsnorm(x_want, weight.double().cpu(), 1e-5), torch.bfloat16)


def test_gemm_in_slices_refuses_what_it_does_not_take():
    ops = _ops()
    a = torch.zeros(65, 64, dtype=torch.bfloat16, device=DEV)
    w = torch.zeros(64, 64, dtype=torch.bfloat16, device=DEV)
    assert not ops.gemm_splitk_supported(a, w)                        # more than 64 rows
    assert not ops.gemm_splitk_supported(a[:8, :60], w[:, :60])       # K no multiple of 8
    assert not ops.gemm_splitk_supported(a[:8].float(), w.float())
    with pytest.raises(ops.KernelError):
        ops.gemm_splitk(a, w, torch.empty(65 * 64, device=DEV), 1)
    with pytest.raises(ops.KernelError):                              # a slice would be empty: 1 chunk, 2 slices
        ops.gemm_splitk(a[:8], w, torch.empty(2 * 8 * 64, device=DEV), 2)
    assert not ops.gemm_splitk_pays(16, 2304, 2304) and not ops.gemm_splitk_pays(65, 2304, 2304)
    assert not ops.gemm_splitk_pays(32, 200, 344)                     # too few blocks for the chip


def test_the_device_peak_measurements_run():
    """The kernels that measure what the matrix cores and the memory deliver when nothing else is done: they run, and
    their figures are of the right order (not a check of the hardware: bounds far from the expected 2,400 and 6)."""
    from infinicore_infer_amd.kernels import peaks
    assert 500 < peaks.mfma_bf16_tflops(iters=2000, blocks_per_unit=4) < 5100
    assert 1.0 < peaks.read_tbs(megabytes=512, blocks_per_unit=8) < 16.5


# ---------------------------------------------------------------------------
# long contexts: the key counts and split counts that the benchmark's steps run with
# ---------------------------------------------------------------------------
def _paged_fast(k, v, page_size, dtype, seed=0, extra_pages=5):
    """As _paged, without a loop over the tokens: shuffled pages, unused rows NaN."""
    t, nkvh, dh = k.shape
    n_pages = (t + page_size - 1) // page_size
    g = torch.Generator().manual_seed(seed)
    perm = torch.randperm(n_pages + extra_pages, generator=g)[:n_pages]
    pad = n_pages * page_size - t

    def plane(x):
        x = torch.cat([x.to(dtype), torch.full((pad, nkvh, dh), float("nan")).to(dtype)]) if pad else x.to(dtype)
        out = torch.full((n_pages + extra_pages, nkvh, page_size, dh), float("nan")).to(dtype)
        out[perm] = x.reshape(n_pages, page_size, nkvh, dh).permute(0, 2, 1, 3)
        return out
    return plane(k), plane(v), perm.to(torch.int32)


@pytest.mark.parametrize("n_split", [8, 16, 32])
@pytest.mark.parametrize("keys", [4100, 16500])
@pytest.mark.parametrize("dtype,nh,nkvh,dh,page", [(torch.bfloat16, 6, 6, 64, 64), (torch.bfloat16, 6, 2, 64, 16),
                                                   (torch.bfloat16, 16, 1, 128, 64), (torch.float32, 4, 4, 64, 64),
                                                   (torch.float32, 4, 2, 128, 32)])
def test_attention_decode_over_long_contexts(dtype, nh, nkvh, dh, page, keys, n_split):
    """Single-token rows over 4,100 and 16,500 keys in 8, 16 and 32 splits (what the cost model chooses for the
    benchmark's steps).  Random rows against the plain attention; and rows that must find ONE key: query i and key
    p_i carry a large component along a direction of their own, so row i's output is value row p_i or the kernel has
    missed that key.  The keys to find lie at the first and last position, at page edges and on both sides of every
    boundary between two splits."""
    ops = _ops()
    g = torch.Generator().manual_seed(keys + n_split)
    scale = 1.0 / math.sqrt(dh)
    per = (keys + n_split - 1) // n_split
    needles = sorted({0, 1, page - 1, page, keys - 1, keys - 2, keys - page, keys // 2}
                     | {min(keys - 1, s * per + o) for s in range(1, n_split, max(1, n_split // 8)) for o in (-1, 0)})[:dh // 2]
    k = torch.randn(keys, nkvh, dh, generator=g) * 0.5
    v = torch.randn(keys, nkvh, dh, generator=g)
    n_rand = 5
    q = torch.randn(n_rand + len(needles), nh, dh, generator=g) * 0.5
    q[n_rand:] *= 0.05
    for i, p in enumerate(needles):            # direction i: element 2 i of every head
        k[p, :, 2 * i] = 30.0
        q[n_rand + i, :, 2 * i] = 30.0         # score 900 / sqrt(dh) >= 79 against the others' few units
    kc, vc, bt = _paged_fast(k, v, page, dtype, seed=keys)
    R = q.shape[0]
    # the random rows see contexts of different lengths; the others see all keys
    ctx = [keys, keys - 1, keys - page, keys // 3, page + 1][:n_rand] + [keys] * len(needles)
    btd = bt[None].repeat(R, 1).contiguous().to(DEV)
    tr = torch.arange(R, dtype=torch.int32, device=DEV)
    ps = torch.tensor([c - 1 for c in ctx], dtype=torch.int32, device=DEV)
    qd = q.to(dtype).reshape(R, nh * dh).to(DEV)
    out = torch.zeros_like(qd)
    pa = torch.empty(R * nh * n_split * dh, device=DEV)
    pm = torch.empty(R * nh * n_split * 2, device=DEV)
    ops.attention_decode(qd, out, kc.to(DEV), vc.to(DEV), btd, None, R, tr, ps, pa, pm, nh, nkvh, dh, page, scale, 0, n_split)
    got = out.float().cpu().reshape(R, nh, dh)
    kd, vd = k.to(dtype).to(DEV), v.to(dtype).to(DEV)
    for r in range(n_rand):
        want = P.plain_attention(q[r:r + 1].to(dtype).to(DEV), kd[:ctx[r]], vd[:ctx[r]], scale, ctx[r] - 1)
        _close(got[r], want[0].cpu(), dtype, factor=3)
    for i, p in enumerate(needles):
        want = v[p].to(dtype).float()          # [nkvh, dh]; head h reads kv head h // (nh / nkvh)
        for h in range(nh):
            err = float((got[n_rand + i, h] - want[h // (nh // nkvh)]).abs().max())
            assert err < 0.05, "the key at position %d of %d (%d splits) was not found by head %d: off by %.3g" % (p, keys, n_split, h, err)


@pytest.mark.parametrize("nh,nkvh,dh,page", [(6, 6, 64, 64), (6, 2, 64, 16), (4, 4, 128, 64), (8, 1, 128, 32)])
@pytest.mark.parametrize("past,new,parts", [(0, 4096, None), (0, 4096, (2, 32)), (3584, 512, (4, 16)), (3000, 1096, (3, 22))])
def test_attention_prefill_walks_of_4096_keys(nh, nkvh, dh, page, past, new, parts):
    """A prompt of 4,096 tokens whole (64 key tiles in the longest walk, whole and cut into parts), and portions after a
    long past.  Against the plain attention; and, as above, query rows that must each find one key of their own: at
    position 0, on both sides of tile and part boundaries, and the row's own position (the diagonal)."""
    ops = _ops()
    g = torch.Generator().manual_seed(past + new + nh)
    t = past + new
    scale = 1.0 / math.sqrt(dh)
    k = torch.randn(t, nkvh, dh, generator=g) * 0.5
    v = torch.randn(t, nkvh, dh, generator=g)
    q = torch.randn(new, nh, dh, generator=g) * 0.5
    part_keys = 64 * (parts[1] if parts else 16)
    rows = sorted({0, 1, 127, 128, new - 1, new - 2, new // 2, new - 129})[:8]
    needles = {}
    for i, r in enumerate(rows):               # query row r (position past + r) must find key p
        pos = past + r
        cand = [0, pos, max(0, pos - 1), min(pos, part_keys - 1), min(pos, part_keys), pos // 2, max(0, pos - 64), min(pos, 63)]
        needles[r] = cand[i % len(cand)]
    used = {}
    for i, (r, p) in enumerate(needles.items()):
        if p in used:                          # two rows after the same key share its direction
            d = used[p]
        else:
            d = used[p] = 2 * len(used)
            k[p, :, d] = 30.0
        q[r] *= 0.05
        q[r, :, d] = 30.0
    kc, vc, bt = _paged_fast(k, v, page, torch.bfloat16, seed=t)
    qd = q.to(torch.bfloat16).reshape(new, nh * dh).to(DEV)
    out = torch.zeros_like(qd)
    tile_rows = ops.attention_prefill_tile_rows()
    tiles = []
    for o in range(0, new, tile_rows):
        tiles += [0, o, min(tile_rows, new - o), past + o]
    tl = torch.tensor(tiles, dtype=torch.int32, device=DEV).view(-1, 4)
    btd = bt[None].contiguous().to(DEV)
    if parts:
        scratch = torch.full((ops.attention_prefill_scratch_floats(tl.shape[0], nh, dh, parts[0]),), float("nan"), device=DEV)
        counters = torch.zeros(ops.attention_prefill_counter_ints(), dtype=torch.int32, device=DEV)
        ops.attention_prefill(qd, out, kc.to(DEV), vc.to(DEV), btd, tl, tl.shape[0], nh, nkvh, dh, page, scale, 0, 1,
                              parts=parts[0], part_len=parts[1], scratch=scratch, counters=counters)
        assert int(counters.abs().sum()) == 0
    else:
        ops.attention_prefill(qd, out, kc.to(DEV), vc.to(DEV), btd, tl, tl.shape[0], nh, nkvh, dh, page, scale, 0)
    want = P.plain_attention(q.to(torch.bfloat16).to(DEV), k.to(torch.bfloat16).to(DEV), v.to(torch.bfloat16).to(DEV), scale, past)
    _close(out.float().cpu().reshape(new, nh, dh), want.cpu(), torch.bfloat16, factor=3)
    got = out.float().cpu().reshape(new, nh, dh)
    for r, p in needles.items():
        vp = v[p].to(torch.bfloat16).float()
        for h in range(nh):
            err = float((got[r, h] - vp[h // (nh // nkvh)]).abs().max())
            assert err < 0.05, "query row %d (position %d) did not find the key at position %d: off by %.3g" % (r, past + r, p, err)
