"""Weights by tensor name: dtypes, tying, and the one error that lists everything (CPU)."""
import json
import os

import pytest
import torch
from safetensors.torch import load_file, save_file

import helpers as H
from infinicore_infer_amd.config import config_from_dict
from infinicore_infer_amd.parts import Runtime, build_model
from infinicore_infer_amd.weights import WeightError, random_state_dict, write_random_model


def _model(name, dtype=torch.bfloat16):
    return build_model(config_from_dict(H.CONFIGS[name][0]).model_spec(), Runtime(dtype, "cpu"))


def test_random_folder_loads_and_is_reproducible(tmp_path):
    a = H.make_model_dir(tmp_path, "A", seed=5)
    assert sorted(os.listdir(a)) == ["config.json", "model.safetensors"]
    sd = load_file(os.path.join(a, "model.safetensors"))
    assert "lm_head.weight" not in sd                       # tied: one table
    assert sd["model.embed_tokens.weight"].dtype == torch.bfloat16
    assert abs(float(sd["model.layers.0.mlp.up_proj.weight"].float().std()) - 0.02) < 0.002
    assert torch.all(sd["model.norm.weight"] == 1)
    again = random_state_dict(H.TINY_A, 5, **H.TINY_A_INIT)
    assert all(torch.equal(sd[k], again[k]) for k in sd)
    other = random_state_dict(H.TINY_A, 6, **H.TINY_A_INIT)
    assert not torch.equal(sd["model.embed_tokens.weight"], other["model.embed_tokens.weight"])
    m = _model("A")
    m.load_from_dir(a)
    assert m.head.weight is m.embedding.table               # jiuge.py:182-191, held once
    assert m.layers[0].mixer.w_qkv.shape == (4 * 16 + 2 * 2 * 16, 64)
    assert m.layers[0].mixer_norm.weight.dtype == torch.float32
    assert m.layers[1].feed_forward.w_gate_up.dtype == torch.bfloat16
    b = H.make_model_dir(tmp_path, "B", seed=5)
    mb = _model("B")
    mb.load_from_dir(b)
    assert mb.head.weight is not mb.embedding.table
    assert float(load_file(os.path.join(b, "model.safetensors"))["model.norm.weight"].float().std()) > 0.05


def test_dtype_rules(tmp_path):
    folder = H.make_model_dir(tmp_path, "A", seed=1)
    m32 = _model("A", torch.float32)
    m32.load_from_dir(folder)
    assert m32.embedding.table.dtype == torch.float32 and m32.layers[0].mixer.w_o.dtype == torch.float32
    # a matrix stored in 32-bit stays so in bfloat16 mode
    sd = load_file(os.path.join(folder, "model.safetensors"))
    sd["model.layers.0.self_attn.o_proj.weight"] = sd["model.layers.0.self_attn.o_proj.weight"].float()
    save_file(sd, os.path.join(folder, "model.safetensors"))
    m = _model("A")
    m.load_from_dir(folder)
    assert m.layers[0].mixer.w_o.dtype == torch.float32
    assert m.layers[1].mixer.w_o.dtype == torch.bfloat16


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    folder = H.make_model_dir(tmp_path, "B", seed=2)
    path = os.path.join(folder, "model.safetensors")
    sd = load_file(path)
    del sd["model.layers.1.mlp.down_proj.weight"]
    del sd["model.layers.2.input_layernorm.weight"]
    sd["model.layers.0.self_attn.q_proj.weight"] = sd["model.layers.0.self_attn.q_proj.weight"][:, :-1].contiguous()
    sd["model.layers.0.mlp.extra.weight"] = torch.zeros(3)
    sd["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(16)      # ignorable buffer
    save_file(sd, path)
    with pytest.raises(WeightError) as e:
        _model("B").load_from_dir(folder)
    err = e.value
    assert err.missing == ["model.layers.1.mlp.down_proj.weight", "model.layers.2.input_layernorm.weight"]
    assert err.unexpected == ["model.layers.0.mlp.extra.weight"]
    assert [w[0] for w in err.wrong_shape] == ["model.layers.0.self_attn.q_proj.weight"]
    msg = str(err)
    for s in ("down_proj", "input_layernorm", "extra.weight", "[96, 95]", "[96, 96]"):
        assert s in msg
    assert "inv_freq" not in msg


def test_missing_both_tables_and_no_files(tmp_path):
    folder = H.make_model_dir(tmp_path, "A", seed=3)
    path = os.path.join(folder, "model.safetensors")
    sd = load_file(path)
    del sd["model.embed_tokens.weight"]
    save_file(sd, path)
    with pytest.raises(WeightError) as e:
        _model("A").load_from_dir(folder)
    assert any("embed_tokens" in m for m in e.value.missing)
    os.remove(path)
    with pytest.raises(WeightError):
        _model("A").load_from_dir(folder)


def test_untied_head_only_backs_the_embedding(tmp_path):
    """lm_head.weight alone serves both tables, as jiuge.py:182-186 allows."""
    folder = H.make_model_dir(tmp_path, "A", seed=4)
    path = os.path.join(folder, "model.safetensors")
    sd = load_file(path)
    sd["lm_head.weight"] = sd.pop("model.embed_tokens.weight")
    save_file(sd, path)
    m = _model("A")
    m.load_from_dir(folder)
    assert m.head.weight is m.embedding.table


def test_random_weights_from_the_command_line(tmp_path):
    """python -m infinicore_infer_amd.weights --config .. --seed .. --out ..: the folder it writes equals
    the one the function writes for the same configuration and seed."""
    import subprocess
    import sys
    cfg_file = tmp_path / "cfg.json"
    cfg_file.write_text(json.dumps(H.TINY_B))
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out = tmp_path / "by_cli"
    r = subprocess.run([sys.executable, "-m", "infinicore_infer_amd.weights", "--config", str(cfg_file), "--seed", "5",
                        "--std", "0.05", "--norm-std", "0.1", "--out", str(out)], cwd=root, capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
    ref = write_random_model(str(tmp_path / "by_call"), H.TINY_B, 5, std=0.05, norm_std=0.1)
    a, b = load_file(str(out / "model.safetensors")), load_file(os.path.join(ref, "model.safetensors"))
    assert sorted(a) == sorted(b) and all(torch.equal(a[k], b[k]) for k in a)
    assert json.load(open(out / "config.json"))["vocab_size"] == H.TINY_B["vocab_size"]
