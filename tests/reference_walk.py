"""A second, independent composition of the decoder: a walk through the reference's own buffers, statement by
statement, in numpy float64.  Where ``plain_model.py`` runs whole sequences without a cache and applies the
constants at run time, this one does what the reference does: constants folded into the weights on the host, q/k
rows permuted, one fused QKV and one fused gate/up matrix, a whole-context cache slab per request, steps of
(req_lens, req_pos) with per-request score matrices [nkvh, ngroup * seq_len, total_len], the residual added by the
projection (beta = 1), the last token of each request normalised and projected.  It shares no code with the
engine or with ``plain_model.py``; the two plain implementations pin each other (tests/test_reference_walk.py).

All paths are relative to the reference checkout.  The bodies of the library operators the reference calls
(RMSNorm, RoPE, CausalSoftmax, SwiGLU) are not in the reference: their standard definitions are used, and where a
call site fixes something (argument order, mask alignment, pair layout) the line is cited.
"""
import math

import numpy as np


def _f64(t):
    return t.detach().to("cpu").double().numpy() if hasattr(t, "detach") else np.asarray(t, dtype=np.float64)


class ReferenceWalk:
    def __init__(self, config, state_dict, max_tokens=None):
        # ---- JiugeMetaFromLlama, scripts/jiuge.py:86-136 ------------------------------------------------
        self.scale_input = self.scale_output = self.scale_o = self.scale_down = 1.0
        if (config["model_type"] in ["fm9g", "minicpm"] and "scale_emb" in config and "scale_depth" in config
                and "dim_model_base" in config):                                             # jiuge.py:101-106
            self.scale_input = config["scale_emb"]                                            # :107
            self.scale_output = config["hidden_size"] // config["dim_model_base"]             # :108 (integer division)
            self.scale_o = config["scale_depth"] / math.sqrt(config["num_hidden_layers"])     # :109-111
            self.scale_down = config["scale_depth"] / math.sqrt(config["num_hidden_layers"])  # :112-114
        self.nlayer = config["num_hidden_layers"]
        self.d = config["hidden_size"]
        self.nh = config["num_attention_heads"]
        self.nkvh = config["num_key_value_heads"] if "num_key_value_heads" in config else config["num_attention_heads"]
        self.dh = config["hidden_size"] // config["num_attention_heads"]                      # :126 (no head_dim key)
        self.di = config["intermediate_size"]
        self.dctx = config["max_position_embeddings"] if max_tokens is None else max_tokens   # :128-130
        self.dvoc = config["vocab_size"]
        self.epsilon = config["rms_norm_eps"]
        self.theta = config["rope_theta"] if "rope_theta" in config else 100000.0             # :133
        nlayer, nh, nkvh, dh, d, di = self.nlayer, self.nh, self.nkvh, self.dh, self.d, self.di
        assert nh % nkvh == 0                                                                 # :160
        sd = {k: _f64(v) for k, v in state_dict.items()}

        # ---- JiugeWeightsImpl, scripts/jiuge.py:139-352 (names: LlamaWeightsNaming, :33-77) -----------------
        input_name = "model.embed_tokens.weight" if "model.embed_tokens.weight" in sd else "lm_head.weight"    # :182-186
        output_name = "lm_head.weight" if "lm_head.weight" in sd else "model.embed_tokens.weight"             # :187-191
        self.input_embd = sd[input_name] * self.scale_input                                   # :193-196
        self.output_norm = sd["model.norm.weight"] * self.scale_output                        # :198-200
        self.output_embd = sd[output_name]                                                    # :202 (kept [dvoc, d], viewed transposed)
        self.attn_norm = [sd["model.layers.%d.input_layernorm.weight" % i] for i in range(nlayer)]           # :209-211
        self.attn_qkv = []
        for i in range(nlayer):                                                               # qkv_slices, :217-236
            p = "model.layers.%d.self_attn." % i
            Q = sd[p + "q_proj.weight"].reshape(nh, 2, dh // 2, d).transpose(0, 2, 1, 3)      # .transpose(1, 2)
            K = sd[p + "k_proj.weight"].reshape(nkvh, 2, dh // 2, d).transpose(0, 2, 1, 3)
            V = sd[p + "v_proj.weight"].reshape(nkvh, dh // 2, 2, d)
            self.attn_qkv.append(np.concatenate([Q.reshape(nh * dh, d), K.reshape(nkvh * dh, d), V.reshape(nkvh * dh, d)]))   # :238-240
        self.attn_o = [sd["model.layers.%d.self_attn.o_proj.weight" % i] * self.scale_o for i in range(nlayer)]      # :284-299
        self.ffn_norm = [sd["model.layers.%d.post_attention_layernorm.weight" % i] for i in range(nlayer)]           # :303-305
        self.ffn_gate_up = [np.concatenate([sd["model.layers.%d.mlp.gate_proj.weight" % i],
                                            sd["model.layers.%d.mlp.up_proj.weight" % i]]) for i in range(nlayer)]  # :311-323
        self.ffn_down = [sd["model.layers.%d.mlp.down_proj.weight" % i] * self.scale_down for i in range(nlayer)]     # :335-350

        # ---- getSinTable / getCosTable, src/models/jiuge/jiuge_weight.hpp:134-186 ---------------------------
        half_dh = dh // 2
        self.sin_table = np.empty((self.dctx, half_dh))
        self.cos_table = np.empty((self.dctx, half_dh))
        for i in range(self.dctx):
            for j in range(half_dh):
                angle = i / math.pow(self.theta, j / half_dh)                                  # :141-142
                self.sin_table[i, j] = math.sin(angle)
                self.cos_table[i, j] = math.cos(angle)

    # ---- createKVCache, src/models/jiuge/jiuge_kv_cache.cpp:3-23 ---------------------------------------------
    def create_kv_cache(self):
        shape = (self.dctx, self.nkvh, self.dh)                                               # :9
        return {"k": [np.zeros(shape) for _ in range(self.nlayer)], "v": [np.zeros(shape) for _ in range(self.nlayer)]}

    # ---- the operators the reference calls (bodies are the library's; standard definitions) --------------------
    def _rmsnorm(self, x, w):                      # inference_context.cpp:36-57: rmsnorm(y, x, w, epsilon)
        return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + self.epsilon) * w

    def _rope(self, x, pos_ids):                   # jiuge.cpp:202-203: in place on [ntok, heads, dh], adjacent pairs after the host permutation
        sin = self.sin_table[pos_ids][:, None, :]
        cos = self.cos_table[pos_ids][:, None, :]
        out = np.empty_like(x)
        a, b = x[..., 0::2], x[..., 1::2]
        out[..., 0::2] = a * cos - b * sin
        out[..., 1::2] = a * sin + b * cos
        return out

    @staticmethod
    def _causal_softmax(s):                        # jiuge.cpp:225-226 on [nh, seq_len, total_len]: the last row sees every key
        nh, seq_len, total_len = s.shape
        out = np.zeros_like(s)
        for i in range(seq_len):
            n = total_len - seq_len + i + 1
            row = s[:, i, :n]
            e = np.exp(row - row.max(axis=-1, keepdims=True))
            out[:, i, :n] = e / e.sum(axis=-1, keepdims=True)
        return out

    # ---- inferDeviceBatch, src/models/jiuge/jiuge.cpp:114-298 ----------------------------------------------------
    def infer_batch(self, tokens, req_lens, req_pos, kv_caches, all_rows=False):
        """Logits [nreq, dvoc] of the last token of every request (the rows the sampler reads, :268-278), or with
        ``all_rows`` of every token (forwardBatch, :261-267)."""
        nlayer, d, nh, nkvh, dh, di = self.nlayer, self.d, self.nh, self.nkvh, self.dh, self.di
        ngroup = nh // nkvh                                                                   # :124
        ntok, nreq = len(tokens), len(req_lens)
        batch_pos_ids = []                                                                    # :147-154
        for req in range(nreq):
            for i in range(req_lens[req]):
                batch_pos_ids.append(req_pos[req] + i)
        batch_pos_ids = np.asarray(batch_pos_ids, dtype=np.int64)
        logits_in = np.stack([self.input_embd[tokens[i]] for i in range(ntok)])              # :164-168
        for layer in range(nlayer):                                                           # :195
            logits_out = self._rmsnorm(logits_in, self.attn_norm[layer])                      # :198
            qkv_buf = logits_out @ self.attn_qkv[layer].T                                     # :200
            qkv_rope = qkv_buf.reshape(ntok, nh + nkvh * 2, dh)                               # :144
            qkv_rope[:, :nh] = self._rope(qkv_rope[:, :nh], batch_pos_ids)                    # :202
            qkv_rope[:, nh:nh + nkvh] = self._rope(qkv_rope[:, nh:nh + nkvh], batch_pos_ids)  # :203
            o_buf = np.empty((ntok, nh * dh))
            token_offset = 0
            for req in range(nreq):                                                           # :206
                past_len, seq_len = req_pos[req], req_lens[req]
                total_len = past_len + seq_len
                rows = slice(token_offset, token_offset + seq_len)
                q = qkv_rope[rows, :nh].reshape(seq_len, nkvh, ngroup, dh).transpose(1, 2, 0, 3)        # :211
                k = qkv_rope[rows, nh:nh + nkvh]                                              # :212
                v = qkv_rope[rows, nh + nkvh:]                                                # :213
                kv_caches[req]["k"][layer][past_len:total_len] = k                            # :217
                kv_caches[req]["v"][layer][past_len:total_len] = v                            # :218
                q_gemm = q.reshape(nkvh, ngroup * seq_len, dh)                                # :220, 223 (as intended: this request's rows)
                k_gemm = kv_caches[req]["k"][layer][:total_len].transpose(1, 2, 0)            # :222  [nkvh, dh, total_len]
                qk_gemm = (q_gemm @ k_gemm) * (1.0 / float(math.sqrt(dh)))                    # :223
                qk_softmax = self._causal_softmax(qk_gemm.reshape(nh, seq_len, total_len))    # :225-226
                v_gemm = kv_caches[req]["v"][layer][:total_len].transpose(1, 0, 2)            # :227  [nkvh, total_len, dh]
                attn_val = qk_softmax.reshape(nkvh, ngroup * seq_len, total_len) @ v_gemm     # :228
                o = attn_val.reshape(nkvh, ngroup, seq_len, dh).transpose(2, 0, 1, 3)         # :210, 230: back to [seq_len, nkvh, ngroup, dh]
                o_buf[rows] = o.reshape(seq_len, nh * dh)
                token_offset += seq_len
            logits_in = o_buf @ self.attn_o[layer].T + logits_in                              # :236 (residual = logits_in)
            logits_out = self._rmsnorm(logits_in, self.ffn_norm[layer])                       # :246
            gate_up_buf = logits_out @ self.ffn_gate_up[layer].T                              # :247
            gate_buf, up_buf = gate_up_buf[:, :di], gate_up_buf[:, di:]                       # :191-192
            gate_buf = up_buf * (gate_buf / (1.0 + np.exp(-gate_buf)))                        # :248 swiglu(out = gate_buf, up_buf, gate_buf)
            logits_in = gate_buf @ self.ffn_down[layer].T + logits_in                         # :249
        if all_rows:
            logits_out = self._rmsnorm(logits_in, self.output_norm)                           # :262
            return logits_out @ self.output_embd.T                                            # :264
        last, token_offset = [], 0
        for req in range(nreq):                                                               # :270-277
            token_offset += req_lens[req]
            last.append(self._rmsnorm(logits_in[token_offset - 1:token_offset], self.output_norm)[0])
        return np.stack(last) @ self.output_embd.T                                            # :278
