"""Plain, slow implementation of the MiniCPM/FM9G decoder, written from the
reference's formulas: whole sequences, no cache, one function for each part.
It shares no code with the engine (it imports nothing from the package).

All paths are relative to the reference checkout.  Arithmetic is float64
unless a rounding function ``rnd`` is given; ``rnd`` is applied where the
engine stores an activation in its compute dtype, so that a bfloat16 engine can
be compared with float64 mathematics on the same rounded values.
"""
import math

import torch

F64 = torch.float64


def _ident(x):
    return x


def round_bf16(x):
    """Round to bfloat16 (nearest even, as src/utils.hpp:109-120 does) and back."""
    return x.to(torch.float32).to(torch.bfloat16).to(x.dtype)


# --------------------------------------------------------------------------
# constants                                                scripts/jiuge.py:97-114
# --------------------------------------------------------------------------
def plain_scales(cfg, logit_scale_rule="reference"):
    """scale_input, scale_output, scale_o (= scale_down).  Applied only when all
    three muP keys exist (jiuge.py:101-106); scale_output uses integer division
    (jiuge.py:108)."""
    if all(k in cfg for k in ("scale_emb", "scale_depth", "dim_model_base")):
        s_in = float(cfg["scale_emb"])
        if logit_scale_rule == "reference":
            s_out = float(cfg["hidden_size"] // cfg["dim_model_base"])
        else:
            s_out = float(cfg["dim_model_base"]) / float(cfg["hidden_size"])
        s_res = float(cfg["scale_depth"]) / math.sqrt(cfg["num_hidden_layers"])
        return s_in, s_out, s_res
    return 1.0, 1.0, 1.0


def plain_dims(cfg):
    """nh, nkvh, dh as scripts/jiuge.py:120-126 derives them."""
    nh = cfg["num_attention_heads"]
    nkvh = cfg.get("num_key_value_heads", nh)
    dh = cfg.get("head_dim") or cfg["hidden_size"] // nh
    return nh, nkvh, dh


# --------------------------------------------------------------------------
# parts
# --------------------------------------------------------------------------
def plain_embedding(table, tokens, scale):
    """x_i = E[token_i] * scale_emb.  jiuge.py:193-197 folds the scale into the
    table; src/models/jiuge/jiuge.cpp:164-168 copies one row per token."""
    return table[torch.as_tensor(tokens, dtype=torch.long, device=table.device)].to(F64) * scale


def plain_rmsnorm(x, w, eps):
    """y = x * rsqrt(mean(x^2) + eps) * w, row-wise.  Call sites
    src/models/jiuge/jiuge.cpp:198,246,262; eps is meta.epsilon = rms_norm_eps
    (jiuge.py:132)."""
    x = x.to(F64)
    ms = (x * x).mean(dim=-1, keepdim=True)
    return x / torch.sqrt(ms + eps) * w.to(F64)


def plain_linear(x, w):
    """y = x W^T with W stored [out, in] (jiuge_weight.hpp:51-54 views it
    transposed; inference_context.cpp:189-233)."""
    return x.to(F64) @ w.to(F64).t()


def plain_rope_tables(dh, theta, npos, factors=None, magnitude=1.0, device=None):
    """sin/cos[p, j] of angle p / theta^(j / (dh/2)), j < dh/2
    (src/models/jiuge/jiuge_weight.hpp:134-159, 161-186).  ``factors`` divides
    each pair's frequency and ``magnitude`` multiplies sin and cos (long-context
    scaling; not in the reference, reduces to it with factors 1, magnitude 1)."""
    half = dh // 2
    j = torch.arange(half, dtype=F64)
    inv = 1.0 / torch.pow(torch.tensor(float(theta), dtype=F64), j / half)
    if factors is not None:
        inv = inv / torch.as_tensor(factors, dtype=F64)
    ang = torch.arange(npos, dtype=F64)[:, None] * inv[None, :]
    return (torch.sin(ang) * magnitude).to(device), (torch.cos(ang) * magnitude).to(device)


def plain_longrope(cfg):
    """Which factor array applies and the magnitude on cos/sin for a configured
    context: the long array and sqrt(1 + ln(ratio)/ln(original)) when the
    configured context exceeds the original one, else the short array and 1."""
    rs = cfg.get("rope_scaling")
    if not rs:
        return None, 1.0
    orig = rs["original_max_position_embeddings"]
    ratio = cfg["max_position_embeddings"] / orig
    if ratio > 1.0:
        return rs["long_factor"], math.sqrt(1.0 + math.log(ratio) / math.log(orig))
    return rs["short_factor"], 1.0


def permute_rows_to_adjacent_pairs(w, n_heads, dh):
    """The reference's host transform of q_proj/k_proj rows (jiuge.py:217-227):
    reshape [n, 2, dh/2, d] -> transpose(1, 2): new row 2j+half <- old row
    half*dh/2 + j, so that pairs (j, j+dh/2) become adjacent (2j, 2j+1)."""
    d = w.shape[1]
    return w.reshape(n_heads, 2, dh // 2, d).transpose(1, 2).reshape(n_heads * dh, d)


def plain_rope_adjacent(x, positions, sin, cos):
    """Rotate adjacent pairs (2j, 2j+1) of every head by the angle of the token's
    position: (a, b) -> (a cos - b sin, a sin + b cos).  x: [T, n, dh].  Call
    sites jiuge.cpp:202-203."""
    pos = torch.as_tensor(positions, dtype=torch.long, device=x.device)
    s = sin[pos][:, None, :]
    c = cos[pos][:, None, :]
    a = x[..., 0::2]
    b = x[..., 1::2]
    out = torch.empty_like(x)
    out[..., 0::2] = a * c - b * s
    out[..., 1::2] = a * s + b * c
    return out


def plain_attention(q, k, v, scale, past=0, window=None):
    """Causal softmax attention of one request over keys 0..t-1 (jiuge.cpp:206-231).
    q: [s, nh, dh]; k, v: [t, nkvh, dh], t = past + s.  Query row i sees keys
    j <= past + i (jiuge.cpp:225-226: the mask is aligned to the bottom right
    of [s, t]).  Query head h uses key/value head h // (nh/nkvh) (jiuge.cpp:210-213:
    heads are viewed as [nkvh, ngroup]).  scale is 1/sqrt(dh) at jiuge.cpp:223.
    ``window`` (not in the reference): row i sees only the last ``window`` keys."""
    s, nh, dh = q.shape
    t, nkvh, _ = k.shape
    g = nh // nkvh
    out = torch.empty(s, nh, dh, dtype=F64, device=q.device)
    qi = past + torch.arange(s, device=q.device)[:, None]
    kj = torch.arange(t, device=q.device)[None, :]
    allowed = kj <= qi
    if window is not None:
        allowed = allowed & (kj > qi - window)
    for h in range(nh):
        kh = k[:, h // g, :].to(F64)
        vh = v[:, h // g, :].to(F64)
        sc = (q[:, h, :].to(F64) @ kh.t()) * scale
        sc = sc.masked_fill(~allowed, float("-inf"))
        p = torch.softmax(sc, dim=-1)
        out[:, h, :] = p @ vh
    return out


def plain_swiglu(gate, up):
    """up * silu(gate), silu(z) = z * sigmoid(z) (jiuge.cpp:248 calls
    swiglu(out=gate_buf, up_buf, gate_buf))."""
    gate = gate.to(F64)
    return up.to(F64) * gate * torch.sigmoid(gate)


# --------------------------------------------------------------------------
# whole model                                  src/models/jiuge/jiuge.cpp:195-267
# --------------------------------------------------------------------------
def plain_forward(cfg, weights, tokens, rnd=None, logit_scale_rule="reference", window=None, start_pos=0,
                  rows=None):
    """Logits [T, vocab] (float64) of one request's whole token sequence from
    position 0.  ``weights``: tensors by checkpoint name (jiuge.py:33-77); the
    arithmetic runs where they lie (the large shapes are checked with the weights
    on the GPU: the same float64 torch operations, only faster)."""
    rnd = rnd or _ident
    nh, nkvh, dh = plain_dims(cfg)
    L = cfg["num_hidden_layers"]
    eps = cfg["rms_norm_eps"]
    theta = cfg.get("rope_theta", 100000.0)                       # jiuge.py:133
    s_in, s_out, s_res = plain_scales(cfg, logit_scale_rule)
    T = len(tokens)
    positions = list(range(start_pos, start_pos + T))     # start_pos != 0 only to test that distances alone count
    factors, magnitude = plain_longrope(cfg)
    emb_name = "model.embed_tokens.weight"
    head_name = "lm_head.weight"
    emb = weights[emb_name] if emb_name in weights else weights[head_name]      # jiuge.py:182-186
    head = weights[head_name] if head_name in weights else weights[emb_name]    # jiuge.py:187-191
    sin, cos = plain_rope_tables(dh, theta, start_pos + T, factors, magnitude, device=emb.device)

    x = plain_embedding(emb, tokens, s_in)
    for l in range(L):
        p = "model.layers.%d." % l
        h = rnd(plain_rmsnorm(x, weights[p + "input_layernorm.weight"], eps))
        wq = permute_rows_to_adjacent_pairs(weights[p + "self_attn.q_proj.weight"].to(F64), nh, dh)
        wk = permute_rows_to_adjacent_pairs(weights[p + "self_attn.k_proj.weight"].to(F64), nkvh, dh)
        wv = weights[p + "self_attn.v_proj.weight"]
        q = rnd(plain_linear(h, wq)).reshape(T, nh, dh)
        k = rnd(plain_linear(h, wk)).reshape(T, nkvh, dh)
        v = rnd(plain_linear(h, wv)).reshape(T, nkvh, dh)
        q = rnd(plain_rope_adjacent(q, positions, sin, cos))
        k = rnd(plain_rope_adjacent(k, positions, sin, cos))
        a = rnd(plain_attention(q, k, v, 1.0 / math.sqrt(dh), 0, window)).reshape(T, nh * dh)
        x = x + s_res * rnd(plain_linear(a, weights[p + "self_attn.o_proj.weight"]))   # jiuge.cpp:236
        h = rnd(plain_rmsnorm(x, weights[p + "post_attention_layernorm.weight"], eps))
        gate = rnd(plain_linear(h, weights[p + "mlp.gate_proj.weight"]))
        up = rnd(plain_linear(h, weights[p + "mlp.up_proj.weight"]))
        act = rnd(plain_swiglu(gate, up))
        x = x + s_res * rnd(plain_linear(act, weights[p + "mlp.down_proj.weight"]))   # jiuge.cpp:249
    if rows is not None:                       # only these positions' logits (the step function's choice, jiuge.cpp:270-277)
        x = x[torch.as_tensor(rows, dtype=torch.long, device=x.device)]
    h = rnd(plain_rmsnorm(x, weights["model.norm.weight"], eps) * s_out)              # jiuge.py:198-201
    return plain_linear(h, head)                                                       # jiuge.cpp:264


# --------------------------------------------------------------------------
# sampling                      jiuge.h:85-88, jiuge.cpp:279-287 (op body external)
# --------------------------------------------------------------------------
def plain_sample(logits, temperature, top_k, top_p, u):
    """One token from raw logits.  Greedy when temperature == 0 or top_k == 1
    (jiuge.h:85-88); ties go to the lowest index.  Otherwise: divide by the
    temperature, keep every value >= the k-th largest (k = 0 or k >= V keeps
    all), softmax, keep the most probable tokens up to and including the one
    with which the kept mass reaches top_p (equal values are kept together),
    then walk the kept tokens in vocabulary order and return the first (of
    non-zero mass) whose cumulated mass reaches u * total."""
    z = torch.as_tensor(logits, dtype=F64)
    V = z.numel()
    if temperature == 0 or top_k == 1:
        return int(torch.argmax(z))          # first maximal index
    z = z / temperature
    keep = torch.ones(V, dtype=torch.bool)
    if 0 < top_k < V:
        kth = torch.sort(z, descending=True).values[top_k - 1]
        keep &= z >= kth
    p = torch.where(keep, torch.exp(z - z[keep].max()), torch.zeros_like(z))
    total = p.sum()
    if top_p < 1.0:
        vals, _ = torch.sort(p, descending=True)
        csum = torch.cumsum(vals, 0)
        idx = int(torch.searchsorted(csum, top_p * total).clamp(max=V - 1))
        thr = vals[idx]
        keep &= p >= thr
        p = torch.where(keep, p, torch.zeros_like(p))
        total = p.sum()
    target = u * total
    csum = torch.cumsum(p, 0)
    cand = torch.nonzero((csum >= target) & keep & (p > 0))
    if cand.numel() == 0:
        return int(torch.nonzero(keep)[-1])
    return int(cand[0])


def plain_generate(cfg, weights, prompt, n_new, rnd=None):
    """Greedy continuation by recomputing the whole sequence every step."""
    toks = list(prompt)
    for _ in range(n_new):
        logits = plain_forward(cfg, weights, toks, rnd=rnd)
        toks.append(int(torch.argmax(logits[-1])))
    return toks[len(prompt):]
