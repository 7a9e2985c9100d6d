"""Configuration and the architecture registry (CPU)."""
import json
import math

import pytest

import helpers as H
from infinicore_infer_amd.config import (ConfigError, MiniCPMConfig, config_from_dict, config_from_dir,
                                         register_architecture, registered_architectures)


def test_tiny_a_values():
    c = config_from_dict(H.TINY_A)
    assert isinstance(c, MiniCPMConfig)
    assert (c.num_attention_heads, c.num_key_value_heads, c.head_dim) == (4, 2, 16)
    assert c.scale_emb == 12 and c.mup
    assert c.residual_scale == pytest.approx(1.4 / math.sqrt(2))          # scripts/jiuge.py:109-114
    assert c.logit_scale == 4.0                                           # 64 // 16, scripts/jiuge.py:108
    assert c.eos_token_id == [2]
    assert config_from_dict(H.TINY_A, logit_scale_rule="mup").logit_scale == pytest.approx(0.25)


def test_defaults_follow_the_reference():
    cfg = {k: v for k, v in H.TINY_B.items() if k not in ("num_key_value_heads", "rope_theta", "scale_emb")}
    c = config_from_dict(cfg)
    assert c.num_key_value_heads == c.num_attention_heads                 # jiuge.py:121-125
    assert c.rope_theta == 100000.0                                       # jiuge.py:133
    assert not c.mup and c.scale_emb == 1.0 and c.residual_scale == 1.0 and c.logit_scale == 1.0   # jiuge.py:97-106
    assert c.eos_token_id == [1, 3]
    assert c.head_dim == 96 // 3


def test_every_size_comes_from_config_json():
    spec = config_from_dict(H.TINY_C).model_spec()
    assert len(spec.layers) == 2 and spec.vocab_size == 331 and spec.hidden_size == 200
    att = spec.layers[1].mixer.params
    assert (att["num_heads"], att["num_kv_heads"], att["head_dim"]) == (6, 2, 64)
    assert att["softmax_scale"] == pytest.approx(1 / 8)
    assert att["position_encoding"].params["scaling"]["original_max_position_embeddings"] == 128
    assert spec.layers[0].feed_forward.params["intermediate_size"] == 344
    assert spec.layers[0].mixer_norm.params["eps"] == 1e-5
    assert spec.embedding.params["scale"] == 4.0 and spec.head.params["logit_scale"] == 4.0
    assert [e.layer for e in spec.schedule] == [0, 1] and spec.num_cache_slots() == 2
    assert spec.layers[0].mixer.name == "model.layers.0.self_attn."


def test_missing_and_bad_keys_are_named():
    cfg = dict(H.TINY_A)
    del cfg["rms_norm_eps"], cfg["vocab_size"]
    with pytest.raises(ConfigError) as e:
        config_from_dict(cfg)
    assert "rms_norm_eps" in str(e.value) and "vocab_size" in str(e.value)
    with pytest.raises(ConfigError):
        config_from_dict(dict(H.TINY_A, num_key_value_heads=3))
    with pytest.raises(ConfigError):
        config_from_dict(dict(H.TINY_A, hidden_act="gelu"))
    with pytest.raises(ConfigError):
        config_from_dict(dict(H.TINY_C, rope_scaling=dict(H.TINY_C["rope_scaling"], short_factor=[1.0] * 3)))
    with pytest.raises(ConfigError):
        config_from_dict(dict(H.TINY_C, rope_scaling={"type": "yarn"}))
    with pytest.raises(ConfigError) as e:      # the reference's integer width ratio would be 0: all logits 0
        config_from_dict(dict(H.TINY_A, dim_model_base=H.TINY_A["hidden_size"] + 1))
    assert "dim_model_base" in str(e.value)


def test_registry_lookup_and_unknown_architecture():
    assert {"minicpm", "fm9g"} <= set(registered_architectures())
    assert isinstance(config_from_dict(dict(H.TINY_A, model_type="x", architectures=["FM9GForCausalLM"])),
                      MiniCPMConfig)
    with pytest.raises(ConfigError) as e:
        config_from_dict(dict(H.TINY_A, model_type="llama", architectures=["LlamaForCausalLM"]))
    assert "minicpm" in str(e.value)


def test_registering_another_architecture():
    class Other:
        @classmethod
        def from_dict(cls, cfg, **kw):
            return cls()

    register_architecture(["other-arch-for-test"], Other)
    assert isinstance(config_from_dict({"model_type": "other-arch-for-test"}), Other)


def test_round_trip_through_a_folder(tmp_path):
    c = config_from_dict(H.TINY_C)
    (tmp_path / "config.json").write_text(json.dumps(c.to_dict()))
    c2 = config_from_dir(str(tmp_path))
    assert c2 == c
    capped = config_from_dir(str(tmp_path), max_tokens=99)                                 # jiuge.py:128-130
    assert capped.max_positions == 99 and capped.model_spec().max_positions == 99
    assert capped.max_position_embeddings == 512 and c.max_positions == 512
    with pytest.raises(ConfigError):
        config_from_dir(str(tmp_path / "nowhere"))


def test_a_cap_on_the_context_changes_no_rotary_value():
    """The cap bounds positions and table length; which longrope factors apply and the magnitude of
    cos/sin follow the checkpoint's own context length.  (TINY_C: 512 configured, 128 original, so the
    long factors and a magnitude above 1 apply; a cap of 100 lies below the original length.)"""
    import torch
    from infinicore_infer_amd.parts.rotary import rotary_tables
    full = config_from_dict(H.TINY_C).model_spec().layers[0].mixer.params["position_encoding"].params
    capped = config_from_dict(H.TINY_C, max_tokens=100).model_spec().layers[0].mixer.params["position_encoding"].params
    assert capped["max_positions"] == 100 and capped["model_max_positions"] == 512
    cos_f, sin_f = rotary_tables(**full)
    cos_c, sin_c = rotary_tables(**capped)
    assert cos_c.shape[0] == 100
    assert torch.equal(cos_c, cos_f[:100]) and torch.equal(sin_c, sin_f[:100])
    assert float(cos_f[0].max()) > 1.0                      # the magnitude factor is in
    # what the mistake would give: factors and magnitude chosen from the cap
    cos_w, _ = rotary_tables(**dict(capped, model_max_positions=100))
    assert not torch.equal(cos_w, cos_c)


def test_torch_dtype_names_the_default_compute_dtype():
    assert config_from_dict(H.TINY_A).default_dtype == "bfloat16"
    assert config_from_dict(dict(H.TINY_A, torch_dtype="float32")).default_dtype == "float32"
    assert config_from_dict(dict(H.TINY_A, torch_dtype="float16")).default_dtype == "bfloat16"
    with pytest.raises(ConfigError):
        config_from_dict(dict(H.TINY_A, torch_dtype="int8"))
