"""Configuration and registry (CPU)."""
import json
import math

import pytest

import qwen_engine_amd  # noqa: F401
from qwen_engine_amd.config import (ConfigError, Qwen3Config, config_from_dict, config_from_folder,
                                    known_architectures, register_architecture, unregister_architecture)
from qwen_engine_amd.config.engine_config import EngineConfig
from tiny import TINY_A, TINY_B, TINY_C


def test_reads_every_size_from_the_dictionary():
    a, b = Qwen3Config.from_dict(TINY_A), Qwen3Config.from_dict(TINY_B)
    assert (a.hidden_size, a.num_attention_heads, a.num_key_value_heads, a.head_dim) == (64, 4, 2, 16)
    assert (b.hidden_size, b.num_attention_heads, b.num_key_value_heads, b.head_dim) == (96, 6, 1, 32)
    assert a.tie_word_embeddings and not b.tie_word_embeddings
    assert a.rms_norm_eps == 1e-6 and b.rms_norm_eps == 1e-5
    # rope_parameters.rope_theta is read before rope_theta (reference config.py:23,35)
    assert b.rope_theta == 1e6
    d = dict(TINY_A, rope_parameters={"rope_theta": 123.0})
    assert Qwen3Config.from_dict(d).rope_theta == 123.0


def test_no_size_has_a_default():
    for key in ("vocab_size", "hidden_size", "intermediate_size", "num_hidden_layers", "num_attention_heads",
                "num_key_value_heads", "head_dim", "max_position_embeddings", "rms_norm_eps",
                "tie_word_embeddings", "rope_theta"):
        d = dict(TINY_A)
        d.pop(key)
        with pytest.raises(ConfigError) as e:
            Qwen3Config.from_dict(d)
        assert key in str(e.value)


def test_all_missing_keys_are_listed_together():
    d = dict(TINY_A)
    d.pop("head_dim")
    d.pop("vocab_size")
    with pytest.raises(ConfigError) as e:
        Qwen3Config.from_dict(d)
    assert "head_dim" in str(e.value) and "vocab_size" in str(e.value)


def test_rejects_what_is_not_modelled():
    with pytest.raises(ConfigError):
        Qwen3Config.from_dict(dict(TINY_A, num_attention_heads=5))          # 5 % 2 != 0
    with pytest.raises(ConfigError):
        Qwen3Config.from_dict(dict(TINY_A, head_dim=15))
    with pytest.raises(ConfigError):
        Qwen3Config.from_dict(dict(TINY_A, rope_scaling={"rope_type": "yarn", "factor": 4.0}))
    with pytest.raises(ConfigError):
        Qwen3Config.from_dict(dict(TINY_A, use_sliding_window=True, sliding_window=64))
    # the keys being present but off is fine
    Qwen3Config.from_dict(dict(TINY_A, rope_scaling=None, use_sliding_window=False, sliding_window=None))


def test_registry_maps_the_architecture_name():
    assert "Qwen3ForCausalLM" in known_architectures()
    assert isinstance(config_from_dict(TINY_B), Qwen3Config)
    with pytest.raises(ConfigError) as e:
        config_from_dict(dict(TINY_A, architectures=["NoSuchModel"]))
    assert "NoSuchModel" in str(e.value) and "Qwen3ForCausalLM" in str(e.value)
    with pytest.raises(ConfigError):
        config_from_dict({k: v for k, v in TINY_A.items() if k != "architectures"})
    marker = object()
    register_architecture("ToyArch", lambda d: marker)
    try:
        assert config_from_dict({"architectures": ["ToyArch"]}) is marker
    finally:
        unregister_architecture("ToyArch")


def test_round_trip_through_config_json(tmp_path):
    c = Qwen3Config.from_dict(dict(TINY_C, eos_token_id=[7, 9]))
    (tmp_path / "config.json").write_text(json.dumps(c.to_dict()))
    again = config_from_folder(str(tmp_path))
    assert again == c
    assert again.eos_token_ids == (7, 9)


def test_model_spec_carries_the_constants():
    c = Qwen3Config.from_dict(TINY_B)
    spec = c.to_model_spec()
    assert len(spec.layers) == 3 and [e.layer for e in spec.schedule] == [0, 1, 2]
    att = spec.layers[0].mixer
    assert att.scale == pytest.approx(1 / math.sqrt(32))        # reference config.py:46
    assert att.qk_norm_eps == 1e-5 and not att.qkv_bias             # q/k norm iff no bias (model.py:204-206)
    assert att.position.theta == 1e6 and att.position.rotary_dim == 32
    assert att.position.max_positions == 640
    biased = Qwen3Config.from_dict(dict(TINY_B, attention_bias=True)).to_model_spec()
    assert biased.layers[0].mixer.qk_norm_eps is None and biased.layers[0].mixer.qkv_bias
    assert spec.layers[1].ffn.intermediate_size == 160
    assert not spec.tie_head and Qwen3Config.from_dict(TINY_A).to_model_spec().tie_head


def test_engine_config_page_count_follows_the_reference():
    e = EngineConfig(max_num_seqs=4, max_model_len=256, block_size=16)
    assert e.pages_per_group() == 64                                # main.py:19-23
    assert EngineConfig(num_blocks=7).pages_per_group() == 7
    with pytest.raises(ValueError):
        EngineConfig(dtype="float16").validate()


def test_pool_sized_from_free_memory():
    """Without num_blocks and with gpu_memory_fraction the pool takes that fraction of the memory that is free
    after the weights, less what recorded steps may hold; the reference's formula (main.py:23) otherwise."""
    from qwen_engine_amd.config import EngineConfig
    cfg = EngineConfig(max_num_seqs=4, max_model_len=256, block_size=16)
    assert cfg.pages_per_group() == 4 * 16                                     # main.py:23
    assert EngineConfig(num_blocks=7, gpu_memory_fraction=0.5).pages_per_group(1 << 40, 4096) == 7   # an explicit number wins
    cfg = EngineConfig(max_model_len=256, block_size=16, gpu_memory_fraction=0.5, graph_memory_bytes=1 << 30)
    per_page = 28 * 2 * 8 * 128 * 2 * 16                                        # bytes of a page through 28 layers
    assert cfg.pages_per_group(10 << 30, per_page) == ((10 << 30) // 2 - (1 << 30)) // per_page
    with pytest.raises(ValueError):
        cfg.pages_per_group()                                                   # needs the two numbers
    with pytest.raises(ValueError):
        cfg.pages_per_group(2 << 30, per_page)                                  # half of 2 GiB less 1 GiB: nothing left
    with pytest.raises(ValueError):
        EngineConfig(gpu_memory_fraction=1.5).validate()
