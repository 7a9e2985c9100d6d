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


def _numpy_standard_normal(seed, name, n):
    """The draw written out a second time, with numpy's unsigned integers: two splitmix64-finalised words per element,
    eight 16-bit uniforms, their centred sum times sqrt(12 / 8)."""
    import hashlib
    import numpy as np
    key = int.from_bytes(hashlib.sha256(("%d:%s" % (seed, name)).encode()).digest()[:8], "little")
    i = np.arange(n, dtype=np.uint64)
    total = np.zeros(n, dtype=np.int64)
    with np.errstate(over="ignore"):
        for word in (0, 1):
            x = i * np.uint64(0x9E3779B97F4A7C15) + np.uint64((key + word * 0x94D049BB133111EB) % (1 << 64))
            x ^= x >> np.uint64(30)
            x *= np.uint64(0xBF58476D1CE4E5B9)
            x ^= x >> np.uint64(27)
            x *= np.uint64(0x94D049BB133111EB)
            x ^= x >> np.uint64(31)
            for field in range(4):
                total += ((x >> np.uint64(16 * field)) & np.uint64(0xFFFF)).astype(np.int64)
    return ((total - (4 * 65536 - 4)).astype(np.float64) * ((1.5 ** 0.5) / 65536.0)).astype(np.float32)


def test_a_random_value_depends_on_seed_name_and_index_only(monkeypatch):
    from infinicore_infer_amd.weights import random_init, standard_normal
    name = "model.layers.3.mlp.up_proj.weight"
    z = standard_normal(7, name, 200000)
    assert torch.equal(z, torch.from_numpy(_numpy_standard_normal(7, name, 200000)))
    # close to a standard normal: mean, variance, fourth moment (Irwin-Hall with n = 8 has kurtosis 3 - 0.15), tails
    assert abs(float(z.mean())) < 0.01 and abs(float(z.var()) - 1.0) < 0.01
    assert abs(float((z ** 4).mean()) - 2.85) < 0.1 and 3.5 < float(z.abs().max()) < 4.9
    # a prefix is a prefix, whatever the pieces it is drawn in
    monkeypatch.setattr(random_init, "_CHUNK_CPU", 777)
    assert torch.equal(standard_normal(7, name, 5000), z[:5000])
    # other seed, other name: other values, uncorrelated
    for other in (standard_normal(8, name, 200000), standard_normal(7, name + "x", 200000)):
        assert abs(float((other * z).mean())) < 0.01
    # neighbouring elements are uncorrelated too
    assert abs(float((z[1:] * z[:-1]).mean())) < 0.01


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


def test_unexpected_dtypes_are_refused_by_tensor_name(tmp_path):
    """A matrix or a norm weight stored as integers or 8-bit floats (a quantized checkpoint) is an
    error that names the tensor, together with whatever else is wrong."""
    folder = H.make_model_dir(tmp_path, "A", seed=3)
    path = os.path.join(folder, "model.safetensors")
    sd = load_file(path)
    sd["model.layers.0.mlp.up_proj.weight"] = torch.zeros(160, 64, dtype=torch.int8)
    sd["model.layers.1.input_layernorm.weight"] = torch.ones(64, dtype=torch.int32)
    if hasattr(torch, "float8_e4m3fn"):
        sd["model.layers.1.self_attn.o_proj.weight"] = torch.zeros(64, 64).to(torch.float8_e4m3fn)
    del sd["model.norm.weight"]
    save_file(sd, path)
    with pytest.raises(WeightError) as e:
        _model("A").load_from_dir(folder)
    names = [w[0] for w in e.value.wrong_dtype]
    assert "model.layers.0.mlp.up_proj.weight" in names and "model.layers.1.input_layernorm.weight" in names
    assert e.value.missing == ["model.norm.weight"]
    msg = str(e.value)
    assert "I8" in msg and "I32" in msg and "up_proj" in msg
    if hasattr(torch, "float8_e4m3fn"):
        assert "model.layers.1.self_attn.o_proj.weight" in names
    # float16 is a floating-point type: converted to the compute dtype, not refused
    folder2 = H.make_model_dir(tmp_path, "B", seed=3)
    sd = load_file(os.path.join(folder2, "model.safetensors"))
    sd = {k: v.to(torch.float16) for k, v in sd.items()}
    save_file(sd, os.path.join(folder2, "model.safetensors"))
    m = _model("B")
    m.load_from_dir(folder2)
    assert m.layers[0].mixer.w_o.dtype == torch.bfloat16 and m.final_norm.weight.dtype == torch.float32


def test_tied_in_the_configuration_but_both_tensors_present(tmp_path):
    """Presence decides which tensor backs which table (scripts/jiuge.py:182-191).  When the
    configuration ties them and the files still hold both: equal tensors are kept once, different ones
    are an error (one of them would silently be ignored otherwise)."""
    folder = H.make_model_dir(tmp_path, "A", seed=4)
    path = os.path.join(folder, "model.safetensors")
    sd = load_file(path)
    sd["lm_head.weight"] = sd["model.embed_tokens.weight"].clone()
    save_file(sd, path)
    m = _model("A")
    m.load_from_dir(folder)
    assert m.head.weight is m.embedding.table or m.head.weight.data_ptr() == m.embedding.table.data_ptr()
    sd["lm_head.weight"] = sd["model.embed_tokens.weight"] * 2
    save_file(sd, path)
    with pytest.raises(WeightError) as e:
        _model("A").load_from_dir(folder)
    assert "lm_head.weight" in str(e.value) and "differ" in str(e.value)
    # not tied in the configuration: both are used as they are
    cfg = dict(H.TINY_A, tie_word_embeddings=False)
    m2 = build_model(config_from_dict(cfg).model_spec(), Runtime(torch.bfloat16, "cpu"))
    m2.load_from_dir(folder)
    assert torch.equal(m2.head.weight, sd["lm_head.weight"]) and torch.equal(m2.embedding.table, sd["model.embed_tokens.weight"])


def test_one_allocation_and_fused_projections_without_a_copy(tmp_path):
    """All tensors are views of one allocation; q, k, v (and gate, up) lie one after the other, so the
    fused projection matrices are views too and equal the concatenation of the stored tensors."""
    from infinicore_infer_amd.weights import loader
    folder = H.make_model_dir(tmp_path, "C", seed=7)
    sd = load_file(os.path.join(folder, "model.safetensors"))
    m = _model("C")
    m.load_from_dir(folder)
    base = m.embedding.table.untyped_storage().data_ptr()
    for p in m.all_parts():
        for k, v in vars(p).items():
            if isinstance(v, torch.Tensor) and k not in ("cos", "sin"):      # rotary tables are no weights
                assert v.untyped_storage().data_ptr() == base
                assert (v.data_ptr() - base) % 256 == 0        # every tensor (and pack) starts on a 256-byte boundary
    for i, layer in enumerate(m.layers):
        n = "model.layers.%d." % i
        want = torch.cat([sd[n + "self_attn.%s_proj.weight" % x] for x in "qkv"], 0)
        assert torch.equal(layer.mixer.w_qkv, want) and layer.mixer.w_qkv.is_contiguous()
        want = torch.cat([sd[n + "mlp.gate_proj.weight"], sd[n + "mlp.up_proj.weight"]], 0)
        assert torch.equal(layer.feed_forward.w_gate_up, want)
        assert torch.equal(layer.mixer_norm.weight, sd[n + "input_layernorm.weight"].float())
    assert loader.last_load_report["bytes"] >= sum(v.numel() * 2 for v in sd.values())
    assert loader.last_load_report["seconds"] > 0
    # q stored in 32-bit, k and v not: no common layout, the part copies them together in float32
    sd["model.layers.0.self_attn.q_proj.weight"] = sd["model.layers.0.self_attn.q_proj.weight"].float()
    save_file(sd, os.path.join(folder, "model.safetensors"))
    m = _model("C")
    m.load_from_dir(folder)
    assert m.layers[0].mixer.w_qkv.dtype == torch.float32 and m.layers[1].mixer.w_qkv.dtype == torch.bfloat16
