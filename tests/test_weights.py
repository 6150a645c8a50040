"""Weights by tensor name and the random-weights mode (CPU)."""
import json
import os

import pytest
import torch
from safetensors.torch import load_file, save_file

import qwen_engine_amd  # noqa: F401
from qwen_engine_amd.config import Qwen3Config
from qwen_engine_amd.parts import expected_tensors
from qwen_engine_amd.parts.base import Runtime
from qwen_engine_amd.weights import WeightError, random_tensors, read_checked, write_model_folder
from tiny import TINY_A, TINY_B


def test_random_folder_has_config_and_every_tensor(tmp_path):
    cfg = Qwen3Config.from_dict(TINY_B)
    folder = write_model_folder(str(tmp_path / "m"), cfg, seed=3)
    assert sorted(os.listdir(folder)) == ["config.json", "model.safetensors"]
    with open(os.path.join(folder, "config.json")) as f:
        d = json.load(f)
    assert d["architectures"] == ["Qwen3ForCausalLM"] and d["hidden_size"] == 96
    stored = load_file(os.path.join(folder, "model.safetensors"))
    exp = expected_tensors(cfg.to_model_spec())
    assert set(stored) == set(exp)
    assert "lm_head.weight" in stored                        # untied
    for name, info in exp.items():
        assert tuple(stored[name].shape) == tuple(info.shape)
        assert stored[name].dtype == torch.bfloat16
    tied = expected_tensors(Qwen3Config.from_dict(TINY_A).to_model_spec())
    assert "lm_head.weight" not in tied


def test_random_weights_depend_on_seed_and_name_only():
    cfg = Qwen3Config.from_dict(TINY_A)
    a, b, c = random_tensors(cfg, 0), random_tensors(cfg, 0), random_tensors(cfg, 1)
    name = "model.layers.1.mlp.up_proj.weight"
    assert torch.equal(a[name], b[name]) and not torch.equal(a[name], c[name])
    # a model with more layers draws the same values for the tensors they have in common
    bigger = random_tensors(Qwen3Config.from_dict(dict(TINY_A, num_hidden_layers=3)), 0)
    assert torch.equal(a[name], bigger[name])
    assert torch.all(a["model.norm.weight"] == 1)
    n = random_tensors(cfg, 0, norm_std=0.01)["model.norm.weight"].float()
    assert 0 < (n - 1).abs().max() < 0.1
    w = a["model.embed_tokens.weight"].float()
    assert abs(w.std().item() - 0.02) < 0.002


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    cfg = Qwen3Config.from_dict(TINY_A)
    exp = expected_tensors(cfg.to_model_spec())
    t = random_tensors(cfg, 0)
    del t["model.layers.0.self_attn.q_norm.weight"]
    del t["model.norm.weight"]
    t["model.layers.0.self_attn.rotary.inv_freq"] = torch.zeros(8)
    t["model.layers.1.mlp.down_proj.weight"] = torch.zeros(64, 127, dtype=torch.bfloat16)
    os.makedirs(tmp_path / "bad")
    save_file(t, str(tmp_path / "bad" / "model.safetensors"))
    with pytest.raises(WeightError) as e:
        read_checked(str(tmp_path / "bad"), exp)
    err = e.value
    assert err.missing == ["model.layers.0.self_attn.q_norm.weight", "model.norm.weight"]
    assert err.unexpected == ["model.layers.0.self_attn.rotary.inv_freq"]
    assert err.wrong_shape == [("model.layers.1.mlp.down_proj.weight", (64, 127), (64, 128))]
    text = str(err)
    for needle in ("q_norm.weight", "model.norm.weight", "inv_freq", "[64, 127]", "[64, 128]"):
        assert needle in text


def test_untied_model_misses_its_head_and_tied_tolerates_one(tmp_path):
    cfg_b = Qwen3Config.from_dict(TINY_B)
    t = random_tensors(cfg_b, 0)
    del t["lm_head.weight"]
    os.makedirs(tmp_path / "b")
    save_file(t, str(tmp_path / "b" / "model.safetensors"))
    with pytest.raises(WeightError) as e:
        read_checked(str(tmp_path / "b"), expected_tensors(cfg_b.to_model_spec()))
    assert e.value.missing == ["lm_head.weight"]
    cfg_a = Qwen3Config.from_dict(TINY_A)
    t = random_tensors(cfg_a, 0)
    t["lm_head.weight"] = t["model.embed_tokens.weight"].clone()
    os.makedirs(tmp_path / "a")
    save_file(t, str(tmp_path / "a" / "model.safetensors"))
    got = read_checked(str(tmp_path / "a"), expected_tensors(cfg_a.to_model_spec()), tied_head_name="lm_head.weight")
    assert "lm_head.weight" not in got


def test_folder_errors(tmp_path):
    with pytest.raises(ValueError):
        read_checked(str(tmp_path / "nowhere"), {})
    os.makedirs(tmp_path / "empty")
    with pytest.raises(ValueError) as e:
        read_checked(str(tmp_path / "empty"), {})
    assert "safetensors" in str(e.value)


def test_several_files_are_read_by_name(tmp_path):
    cfg = Qwen3Config.from_dict(TINY_A)
    t = random_tensors(cfg, 0)
    names = sorted(t)
    os.makedirs(tmp_path / "s")
    save_file({n: t[n] for n in names[:10]}, str(tmp_path / "s" / "model-00001-of-00002.safetensors"))
    save_file({n: t[n] for n in names[10:]}, str(tmp_path / "s" / "model-00002-of-00002.safetensors"))
    got = read_checked(str(tmp_path / "s"), expected_tensors(cfg.to_model_spec()))
    assert all(torch.equal(got[n], t[n]) for n in names)


def test_placement_keeps_stored_precision():
    cpu = torch.device("cpu")
    bf, f32 = Runtime(cpu, torch.bfloat16), Runtime(cpu, torch.float32)
    m16 = torch.randn(4, 4).to(torch.bfloat16)
    m32 = torch.randn(4, 4)
    table = torch.arange(6, dtype=torch.int64)
    assert bf.place_matrix(m16).dtype == torch.bfloat16
    assert bf.place_matrix(m32).dtype == torch.float32          # stored in 32-bit: stays so
    assert f32.place_matrix(m16).dtype == torch.float32
    assert torch.equal(f32.place_matrix(m16), m16.float())      # exact
    assert bf.place_matrix(table).dtype == torch.int32
    assert bf.place_vector(m16[0]).dtype == torch.float32


def test_tensors_are_read_part_by_part(tmp_path, monkeypatch):
    """read_checked opens the files and checks names and shapes, but reads no tensor; the model then
    asks for each tensor once, part by part (the reference holds the whole checkpoint on the host
    first, utils.py:77-82), and the parts see their tensors under their own names."""
    from qwen_engine_amd.parts import DecoderModel
    from qwen_engine_amd.weights.loader import LazyTensors
    cfg = Qwen3Config.from_dict(TINY_B)
    folder = write_model_folder(str(tmp_path / "m"), cfg, 3)
    spec = cfg.to_model_spec()
    read = []
    real = LazyTensors.__getitem__
    monkeypatch.setattr(LazyTensors, "__getitem__", lambda self, name: (read.append(self._names[name]), real(self, name))[1])
    got = read_checked(folder, expected_tensors(spec))
    assert read == [] and len(got) == len(expected_tensors(spec))
    layer0 = got.subset("model.layers.0.")
    assert "self_attn.q_proj.weight" in layer0 and "mlp.down_proj.weight" in layer0 and read == []
    assert all(not k.startswith("model.") for k in layer0)
    model = DecoderModel(spec)
    model.load(got, Runtime(torch.device("cpu"), torch.float32))
    assert sorted(read) == sorted(expected_tensors(spec))          # every tensor exactly once
    assert read[0] == "model.embed_tokens.weight" and read[-1] == "lm_head.weight"
    t = random_tensors(cfg, 3)
    assert torch.equal(model.blocks[2].mixer.w_o, t["model.layers.2.self_attn.o_proj.weight"].float())
