"""Loading by tensor name, the one error that lists everything wrong, random weights (no GPU)."""
import json
import os

import numpy as np
import pytest
import torch

import helpers
import plain
import hf_cpu_amd
from hf_cpu_amd.config import config_from_dict, read_config
from hf_cpu_amd.status import EngineError
from hf_cpu_amd.weights import SafetensorsFile, load_tensors, write_random_model, write_safetensors


def specs_for(cfg):
    return hf_cpu_amd.Model.from_config(config_from_dict(cfg)).param_specs()


def test_loads_by_name_and_keeps_precisions(tmp_path):
    d = helpers.make_model_dir(str(tmp_path / "f32"), helpers.CONFIG_B, seed=3)
    w = helpers.make_weights(helpers.CONFIG_B, seed=3)
    t32 = load_tensors(d, specs_for(helpers.CONFIG_B), torch.float32, "cpu")
    assert set(t32) == set(w)
    for name, a in w.items():
        assert t32[name].dtype == torch.float32 and np.array_equal(t32[name].numpy(), a)
    # bf16 compute: a tensor stored in 32-bit stays so; vectors are fp32 in any case
    t16 = load_tensors(d, specs_for(helpers.CONFIG_B), torch.bfloat16, "cpu")
    assert all(t.dtype == torch.float32 for t in t16.values())
    d16 = helpers.make_model_dir(str(tmp_path / "bf16"), helpers.CONFIG_B, seed=3, dtype="BF16")
    t = load_tensors(d16, specs_for(helpers.CONFIG_B), torch.bfloat16, "cpu")
    assert t["model.layers.0.mlp.up_proj.weight"].dtype == torch.bfloat16
    assert t["model.layers.0.input_layernorm.weight"].dtype == torch.float32
    assert t["model.layers.0.self_attn.q_proj.bias"].dtype == torch.float32
    want = helpers.bf16_round(w["model.layers.0.mlp.up_proj.weight"])
    assert np.array_equal(t["model.layers.0.mlp.up_proj.weight"].float().numpy(), want)
    wide = load_tensors(d16, specs_for(helpers.CONFIG_B), torch.float32, "cpu")
    assert wide["model.layers.0.mlp.up_proj.weight"].dtype == torch.float32
    assert np.array_equal(wide["model.layers.0.mlp.up_proj.weight"].numpy(), want)


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    cfg = helpers.CONFIG_B
    w = helpers.make_weights(cfg, seed=1)
    del w["model.layers.1.self_attn.k_proj.bias"]
    del w["lm_head.weight"]
    w["model.layers.0.mlp.down_proj.weight"] = w["model.layers.0.mlp.down_proj.weight"].T.copy()
    w["model.norm.weight"] = np.ones(95, np.float32)
    w["model.layers.7.surprise"] = np.ones(3, np.float32)
    d = helpers.make_model_dir(str(tmp_path / "bad"), cfg, 0, weights=w)
    with pytest.raises(EngineError) as e:
        load_tensors(d, specs_for(cfg), torch.float32, "cpu")
    msg = str(e.value)
    assert e.value.code == "EFORMAT"
    assert "missing tensors: " in msg and "model.layers.1.self_attn.k_proj.bias" in msg and "lm_head.weight" in msg
    assert "unexpected tensors: model.layers.7.surprise" in msg
    assert "model.layers.0.mlp.down_proj.weight has shape 256x96, expected 96x256" in msg
    assert "model.norm.weight has shape 95, expected 96" in msg


def test_tied_head_is_optional_and_present_wins(tmp_path):
    cfg = helpers.CONFIG_A                                       # tied
    w = helpers.make_weights(cfg, seed=1)
    d = helpers.make_model_dir(str(tmp_path / "tied"), cfg, 0, weights=w)
    assert "lm_head.weight" not in load_tensors(d, specs_for(cfg), torch.float32, "cpu")
    w["lm_head.weight"] = np.zeros((512, 64), np.float32)
    d2 = helpers.make_model_dir(str(tmp_path / "both"), cfg, 0, weights=w)
    assert "lm_head.weight" in load_tensors(d2, specs_for(cfg), torch.float32, "cpu")     # src/model.c:156-158


def test_container_errors(tmp_path):
    p = tmp_path / "model.safetensors"
    (tmp_path / "config.json").write_text(json.dumps(helpers.CONFIG_A))
    with pytest.raises(EngineError) as e:
        load_tensors(str(tmp_path), specs_for(helpers.CONFIG_A), torch.float32, "cpu")
    assert e.value.code == "EIO"
    p.write_bytes(b"\x05\x00")
    with pytest.raises(EngineError) as e:
        SafetensorsFile(str(p))
    assert e.value.code == "EFORMAT"
    p.write_bytes((1 << 40).to_bytes(8, "little") + b"{}")
    with pytest.raises(EngineError, match="header length"):
        SafetensorsFile(str(p))
    head = json.dumps({"a": {"dtype": "F32", "shape": [4], "data_offsets": [0, 8]}}).encode()
    p.write_bytes(len(head).to_bytes(8, "little") + head + b"\0" * 8)
    with pytest.raises(EngineError, match="does not match"):
        SafetensorsFile(str(p))
    head = json.dumps({"a": {"dtype": "F8_E4M3", "shape": [4], "data_offsets": [0, 4]}}).encode()
    p.write_bytes(len(head).to_bytes(8, "little") + head + b"\0" * 4)
    f = SafetensorsFile(str(p))
    from hf_cpu_amd.parts import ParamSpec
    from hf_cpu_amd.weights import check_tensors
    with pytest.raises(EngineError, match="stored as F8_E4M3"):
        check_tensors(f.entries, [ParamSpec("a", (4,))], "x")


def test_random_weights_folder(tmp_path):
    cfg = config_from_dict(helpers.CONFIG_B)
    d = write_random_model(str(tmp_path / "r"), cfg, seed=5, dtype="bfloat16")
    assert sorted(os.listdir(d)) == ["config.json", "model.safetensors"]
    back = read_config(d)
    assert back.hidden_size == 96 and back.torch_dtype == "bfloat16" and back.sliding_window == 32
    c2, w = plain.read_model(d)                                  # the tests' own reader reads it too
    assert set(w) == {s.name for s in specs_for(helpers.CONFIG_B)}
    m = w["model.layers.1.mlp.gate_proj.weight"]
    assert abs(m.std() - 0.02) < 0.002 and abs(m.mean()) < 0.001
    n = w["model.layers.2.input_layernorm.weight"]
    assert abs(n.mean() - 1.0) < 0.05 and 0.05 < n.std() < 0.15
    assert abs(w["model.layers.0.self_attn.q_proj.bias"].std() - 0.02) < 0.006
    d2 = write_random_model(str(tmp_path / "r2"), cfg, seed=5, dtype="bfloat16")
    assert open(os.path.join(d, "model.safetensors"), "rb").read() == \
        open(os.path.join(d2, "model.safetensors"), "rb").read()
    d3 = write_random_model(str(tmp_path / "r3"), cfg, seed=6, dtype="float32")
    w3 = plain.read_safetensors(os.path.join(d3, "model.safetensors"))
    assert not np.array_equal(w3["model.norm.weight"], w["model.norm.weight"])
    tied = write_random_model(str(tmp_path / "t"), config_from_dict(helpers.CONFIG_A), seed=0)
    assert "lm_head.weight" not in plain.read_safetensors(os.path.join(tied, "model.safetensors"))
    logits = plain.forward(*plain.read_model(tied), [1, 2, 3])
    assert logits.shape == (3, 512) and np.isfinite(logits).all()


def test_random_generator_is_the_stated_rule():
    """The counter-based generator of the random weights, element by element against its statement
    in plain integers (splitmix64's finishing function on key + 2e and key + 2e + 1, the eight 16-bit
    fields added up, one fp32 product); pieces of a tensor equal the whole; the moments are a Gaussian's."""
    from hf_cpu_amd.weights.random_init import random_values, tensor_key
    M = (1 << 64) - 1

    def mix(z):
        z &= M
        z = ((z ^ (z >> 30)) * 0xbf58476d1ce4e5b9) & M
        z = ((z ^ (z >> 27)) * 0x94d049bb133111eb) & M
        return z ^ (z >> 31)
    key = tensor_key(7, 3)
    assert key == mix(7 * 0x9e3779b97f4a7c15 + 3)
    got = random_values(key, 50, "normal", 0.02)
    scale = np.float32(0.02 / np.sqrt(8 * (65536.0 ** 2 - 1) / 12))
    for e in (0, 1, 17, 49):
        a, b = mix(key + 2 * e), mix(key + 2 * e + 1)
        total = sum((w >> s) & 0xffff for w in (a, b) for s in (0, 16, 32, 48))
        assert got[e] == np.float32(total - 262140) * scale
    assert np.array_equal(random_values(key, 20, "normal", 0.02, first=30), got[30:])
    assert np.array_equal(random_values(key, 50, "one_plus_normal", 0.02), np.float32(1.0) + got)
    table = random_values(key, 1000, "table", 37)
    assert table.dtype == np.int32 and table.min() >= 0 and table.max() < 37 and table[5] == mix(key + 10) % 37
    big = random_values(tensor_key(0, 0), 400000, "normal", 1.0).astype(np.float64)
    assert abs(big.mean()) < 0.01 and abs(big.std() - 1.0) < 0.01
    assert abs(np.mean(big ** 4) - 3.0) < 0.2 and np.abs(big).max() < 4.9        # kurtosis 3 - 1.2 / 8
    assert not np.array_equal(random_values(tensor_key(0, 1), 50, "normal", 0.02), random_values(tensor_key(1, 0), 50, "normal", 0.02))


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["bfloat16", "float32"])
def test_random_weights_are_the_same_bits_from_the_file_and_on_the_device(gpu, tmp_path, dtype):
    """``Model.from_random(config, seed)`` (weights made by a kernel) holds what ``Model.from_dir`` loads
    from the folder that ``write_random_model(config, seed)`` wrote: one generator for both."""
    import hf_cpu_amd
    from hf_cpu_amd.kernels import Ops
    from hf_cpu_amd.model import compute_dtype
    cfg = config_from_dict(helpers.CONFIG_B)
    d = write_random_model(str(tmp_path / "r"), cfg, seed=11, dtype=dtype)
    ops = Ops(compute_dtype(dtype), gpu)
    a = hf_cpu_amd.Model.from_dir(d, dtype, ops)
    b = hf_cpu_amd.Model.from_random(cfg, 11, dtype, ops)
    seen = 0
    for la, lb in zip(a._all_parts(), b._all_parts()):
        for name, ta in vars(la).items():
            if isinstance(ta, torch.Tensor):
                tb = getattr(lb, name)
                assert ta.dtype == tb.dtype and torch.equal(ta, tb), f"{type(la).__name__}.{name}"
                seen += 1
    assert seen >= 3 * 6 + 3
    c = hf_cpu_amd.Model.from_random(cfg, 12, dtype, ops)
    assert not torch.equal(c.embedding.table if hasattr(c.embedding, "table") else next(
        t for t in vars(c.embedding).values() if isinstance(t, torch.Tensor)), next(
        t for t in vars(b.embedding).values() if isinstance(t, torch.Tensor)))


def test_writer_round_trip(tmp_path):
    t = {"a": torch.arange(6, dtype=torch.float32).reshape(2, 3), "b": torch.tensor([1.5, -2.0]).bfloat16(),
         "c": torch.tensor([[1, 2], [3, 4]], dtype=torch.int32)}
    p = str(tmp_path / "x.safetensors")
    write_safetensors(p, t, {"k": "v"})
    f = SafetensorsFile(p)
    assert f.metadata == {"k": "v"}
    for k, v in t.items():
        assert torch.equal(f.read(k), v)
