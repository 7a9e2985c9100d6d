"""Typed configuration of the MiniCPM / FM9G decoder, read from config.json.

Keys and defaults follow the reference's reader, scripts/jiuge.py:86-135:
  num_key_value_heads defaults to num_attention_heads      (jiuge.py:121-125)
  head size = hidden_size // num_attention_heads            (jiuge.py:126)
  rope_theta defaults to 100000.0 when absent               (jiuge.py:133)
  eos_token_id is an int or a list                          (jiuge.py:415-418)
  the muP constants apply only when scale_emb, scale_depth and dim_model_base
  are all present, otherwise every scale is 1.0             (jiuge.py:97-114)
    scale_input  = scale_emb
    scale_output = hidden_size // dim_model_base   (integer division, a multiplier
                   on the final norm's weight, jiuge.py:108,198-201)
    scale_o = scale_down = scale_depth / sqrt(num_hidden_layers)
Keys the reference does not read but checkpoints of this family carry are read
too: head_dim, tie_word_embeddings, rope_scaling (longrope), torch_dtype,
bos_token_id, hidden_act.
"""
import math
from dataclasses import dataclass, field, asdict
from typing import List, Optional

from .registry import ConfigError, register_architecture
from .spec import ExecEntry, LayerSpec, ModelSpec, PartSpec, default_schedule

_REQUIRED = (
    "vocab_size", "hidden_size", "num_hidden_layers", "num_attention_heads",
    "intermediate_size", "max_position_embeddings", "rms_norm_eps",
)


@dataclass
class RopeScaling:
    """Long-context rotary scaling ("longrope"): per-pair divisors of the
    rotary frequencies, one array for contexts up to the original length and
    one for longer ones, and a magnitude factor on cos/sin."""
    type: str
    short_factor: List[float]
    long_factor: List[float]
    original_max_position_embeddings: int


@dataclass
class MiniCPMConfig:
    vocab_size: int
    hidden_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    intermediate_size: int
    max_position_embeddings: int
    rms_norm_eps: float
    rope_theta: float = 100000.0
    rope_scaling: Optional[RopeScaling] = None
    scale_emb: float = 1.0
    scale_depth: Optional[float] = None
    dim_model_base: Optional[int] = None
    mup: bool = False
    tie_word_embeddings: Optional[bool] = None
    eos_token_id: List[int] = field(default_factory=list)
    bos_token_id: Optional[int] = None
    torch_dtype: str = "bfloat16"
    model_type: str = "minicpm"
    # "reference": the final hidden state is multiplied by hidden_size // dim_model_base,
    # as scripts/jiuge.py:108,199 does.  "mup": divided by hidden_size / dim_model_base.
    logit_scale_rule: str = "reference"
    # The serving cap on a request's length (the reference's max_tokens argument,
    # scripts/jiuge.py:128-130).  It bounds positions, the rotary tables and the cache; the
    # checkpoint's own max_position_embeddings stays what long-context scaling is derived from.
    context_cap: Optional[int] = None

    # ---- reading ---------------------------------------------------------
    @classmethod
    def from_dict(cls, cfg: dict, max_tokens: Optional[int] = None,
                  logit_scale_rule: str = "reference") -> "MiniCPMConfig":
        missing = [k for k in _REQUIRED if k not in cfg]
        if missing:
            raise ConfigError("config.json lacks required key(s): %s" % ", ".join(missing))
        nh = int(cfg["num_attention_heads"])
        d = int(cfg["hidden_size"])
        if nh <= 0 or d <= 0:
            raise ConfigError("hidden_size and num_attention_heads must be positive")
        nkvh = int(cfg.get("num_key_value_heads") or nh)
        head_dim = int(cfg["head_dim"]) if cfg.get("head_dim") else d // nh
        act = cfg.get("hidden_act", "silu")
        if act != "silu":
            raise ConfigError("hidden_act %r: this architecture's feed-forward is SwiGLU (silu)" % act)
        mup = all(k in cfg for k in ("scale_emb", "scale_depth", "dim_model_base"))
        eos = cfg.get("eos_token_id", [])
        if eos is None:
            eos = []
        if isinstance(eos, int):
            eos = [eos]
        rs = cfg.get("rope_scaling")
        rope_scaling = None
        if rs:
            kind = rs.get("rope_type", rs.get("type"))
            if kind != "longrope":
                raise ConfigError("rope_scaling type %r is not supported (longrope only)" % kind)
            for k in ("short_factor", "long_factor", "original_max_position_embeddings"):
                if k not in rs:
                    raise ConfigError("rope_scaling lacks %r" % k)
            rope_scaling = RopeScaling(
                type=kind,
                short_factor=[float(v) for v in rs["short_factor"]],
                long_factor=[float(v) for v in rs["long_factor"]],
                original_max_position_embeddings=int(rs["original_max_position_embeddings"]))
        out = cls(
            vocab_size=int(cfg["vocab_size"]),
            hidden_size=d,
            num_hidden_layers=int(cfg["num_hidden_layers"]),
            num_attention_heads=nh,
            num_key_value_heads=nkvh,
            head_dim=head_dim,
            intermediate_size=int(cfg["intermediate_size"]),
            max_position_embeddings=int(cfg["max_position_embeddings"]),
            context_cap=int(max_tokens) if max_tokens is not None else None,
            rms_norm_eps=float(cfg["rms_norm_eps"]),
            rope_theta=float(cfg.get("rope_theta", 100000.0)),
            rope_scaling=rope_scaling,
            scale_emb=float(cfg["scale_emb"]) if mup else 1.0,
            scale_depth=float(cfg["scale_depth"]) if mup else None,
            dim_model_base=int(cfg["dim_model_base"]) if mup else None,
            mup=mup,
            tie_word_embeddings=cfg.get("tie_word_embeddings"),
            eos_token_id=[int(e) for e in eos],
            bos_token_id=cfg.get("bos_token_id"),
            torch_dtype=str(cfg.get("torch_dtype", "bfloat16")),
            model_type=str(cfg.get("model_type", "minicpm")),
            logit_scale_rule=logit_scale_rule,
        )
        out.validate()
        return out

    def validate(self) -> None:
        pos = ("vocab_size", "hidden_size", "num_hidden_layers", "num_attention_heads",
               "num_key_value_heads", "head_dim", "intermediate_size", "max_position_embeddings")
        for k in pos:
            if getattr(self, k) <= 0:
                raise ConfigError("%s must be positive, got %r" % (k, getattr(self, k)))
        if self.context_cap is not None and self.context_cap <= 0:
            raise ConfigError("max_tokens (the cap on the context) must be positive, got %r" % (self.context_cap,))
        if self.torch_dtype not in ("bfloat16", "float32", "float16"):
            raise ConfigError("torch_dtype %r: bfloat16, float32 or float16 expected" % (self.torch_dtype,))
        if self.num_attention_heads % self.num_key_value_heads:
            raise ConfigError("num_attention_heads (%d) is not a multiple of num_key_value_heads (%d)"
                              % (self.num_attention_heads, self.num_key_value_heads))
        if self.head_dim % 2:
            raise ConfigError("head_dim (%d) must be even for rotary pairs" % self.head_dim)
        if not (self.rms_norm_eps > 0):
            raise ConfigError("rms_norm_eps must be positive")
        if self.rope_theta <= 0:
            raise ConfigError("rope_theta must be positive")
        if self.mup and self.dim_model_base <= 0:
            raise ConfigError("dim_model_base must be positive")
        if self.logit_scale_rule not in ("reference", "mup"):
            raise ConfigError("logit_scale_rule must be 'reference' or 'mup'")
        if self.mup and self.logit_scale_rule == "reference" and self.hidden_size // self.dim_model_base == 0:
            raise ConfigError("dim_model_base (%d) above hidden_size (%d): the integer ratio that scales the "
                              "logits (hidden_size // dim_model_base) is 0 and every logit would be 0"
                              % (self.dim_model_base, self.hidden_size))
        rs = self.rope_scaling
        if rs is not None:
            half = self.head_dim // 2
            if len(rs.short_factor) != half or len(rs.long_factor) != half:
                raise ConfigError("rope_scaling factors must have head_dim/2 = %d entries" % half)
            if rs.original_max_position_embeddings <= 0:
                raise ConfigError("original_max_position_embeddings must be positive")

    # ---- derived constants -------------------------------------------------
    @property
    def max_positions(self) -> int:
        """Positions a request may reach: the cap when one is given (jiuge.py:128-130), else the
        checkpoint's max_position_embeddings."""
        return self.context_cap if self.context_cap is not None else self.max_position_embeddings

    @property
    def default_dtype(self) -> str:
        """The compute dtype to use when the caller names none: the checkpoint's torch_dtype;
        float16 checkpoints run in bfloat16 (the kernels take bfloat16 and float32)."""
        return "float32" if self.torch_dtype == "float32" else "bfloat16"

    @property
    def residual_scale(self) -> float:
        """scale_depth / sqrt(num_hidden_layers) on each branch (jiuge.py:109-114)."""
        if not self.mup:
            return 1.0
        return self.scale_depth / math.sqrt(self.num_hidden_layers)

    @property
    def logit_scale(self) -> float:
        if not self.mup:
            return 1.0
        if self.logit_scale_rule == "reference":
            return float(self.hidden_size // self.dim_model_base)   # jiuge.py:108
        return float(self.dim_model_base) / float(self.hidden_size)

    # ---- writing -------------------------------------------------------------
    def to_dict(self) -> dict:
        d = {
            "architectures": ["MiniCPMForCausalLM"],
            "model_type": self.model_type,
            "vocab_size": self.vocab_size,
            "hidden_size": self.hidden_size,
            "num_hidden_layers": self.num_hidden_layers,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads,
            "intermediate_size": self.intermediate_size,
            "max_position_embeddings": self.max_position_embeddings,
            "rms_norm_eps": self.rms_norm_eps,
            "rope_theta": self.rope_theta,
            "hidden_act": "silu",
            "torch_dtype": self.torch_dtype,
            "eos_token_id": list(self.eos_token_id),
        }
        if self.head_dim != self.hidden_size // self.num_attention_heads:
            d["head_dim"] = self.head_dim
        if self.mup:
            d["scale_emb"] = self.scale_emb
            d["scale_depth"] = self.scale_depth
            d["dim_model_base"] = self.dim_model_base
        if self.tie_word_embeddings is not None:
            d["tie_word_embeddings"] = bool(self.tie_word_embeddings)
        if self.bos_token_id is not None:
            d["bos_token_id"] = self.bos_token_id
        if self.rope_scaling is not None:
            d["rope_scaling"] = asdict(self.rope_scaling)
        return d

    # ---- the model as data -----------------------------------------------------
    def model_spec(self) -> ModelSpec:
        """Describe the model layer by layer.  Tensor names are the reference's
        (scripts/jiuge.py:33-77)."""
        rotary = PartSpec("rotary", "", {
            "head_dim": self.head_dim,
            "theta": self.rope_theta,
            "max_positions": self.max_positions,
            "model_max_positions": self.max_position_embeddings,
            "scaling": asdict(self.rope_scaling) if self.rope_scaling else None,
        })
        layers = []
        for i in range(self.num_hidden_layers):
            p = "model.layers.%d." % i
            layers.append(LayerSpec(
                block=PartSpec("prenorm_residual", p, {"residual_scale": self.residual_scale}),
                mixer=PartSpec("attention", p + "self_attn.", {
                    "hidden_size": self.hidden_size,
                    "num_heads": self.num_attention_heads,
                    "num_kv_heads": self.num_key_value_heads,
                    "head_dim": self.head_dim,
                    "softmax_scale": 1.0 / math.sqrt(self.head_dim),   # jiuge.cpp:223
                    "window": None,
                    "position_encoding": rotary,
                }),
                mixer_norm=PartSpec("rmsnorm", p + "input_layernorm.", {
                    "size": self.hidden_size, "eps": self.rms_norm_eps}),
                feed_forward=PartSpec("swiglu", p + "mlp.", {
                    "hidden_size": self.hidden_size,
                    "intermediate_size": self.intermediate_size}),
                feed_forward_norm=PartSpec("rmsnorm", p + "post_attention_layernorm.", {
                    "size": self.hidden_size, "eps": self.rms_norm_eps}),
            ))
        return ModelSpec(
            architecture=self.model_type,
            vocab_size=self.vocab_size,
            hidden_size=self.hidden_size,
            max_positions=self.max_positions,
            embedding=PartSpec("embedding", "model.embed_tokens.", {
                "vocab_size": self.vocab_size, "hidden_size": self.hidden_size,
                "scale": self.scale_emb, "fallback_name": "lm_head."}),
            layers=layers,
            schedule=default_schedule(self.num_hidden_layers),
            final_norm=PartSpec("rmsnorm", "model.norm.", {
                "size": self.hidden_size, "eps": self.rms_norm_eps}),
            head=PartSpec("lm_head", "lm_head.", {
                "vocab_size": self.vocab_size, "hidden_size": self.hidden_size,
                "logit_scale": self.logit_scale, "fallback_name": "model.embed_tokens.",
                "tied": bool(self.tie_word_embeddings)}),
            eos_token_ids=list(self.eos_token_id),
            bos_token_id=self.bos_token_id,
        )


register_architecture(["minicpm", "fm9g", "MiniCPMForCausalLM", "FM9GForCausalLM"], MiniCPMConfig)
