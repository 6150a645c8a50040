"""Tiny configurations of the architecture for tests: two that differ in every size
and option, written as model folders with random weights into a temporary place."""
import json
import os

import torch

import qwen_engine_amd  # noqa: F401
from qwen_engine_amd.config import Qwen3Config
from qwen_engine_amd.weights import write_model_folder

# A: 2 layers, width 64, 4 query heads on 2 key/value heads of 16, tied head.
TINY_A = dict(
    architectures=["Qwen3ForCausalLM"], vocab_size=256, hidden_size=64, intermediate_size=128,
    num_hidden_layers=2, num_attention_heads=4, num_key_value_heads=2, head_dim=16,
    max_position_embeddings=512, rms_norm_eps=1e-6, rope_theta=10000.0, tie_word_embeddings=True)
# B: 3 layers, width 96, 6 query heads on 1 key/value head of 32 (query width 192 != 96),
# sizes that are no power of two, other eps and theta, head of its own.
TINY_B = dict(
    architectures=["Qwen3ForCausalLM"], vocab_size=500, hidden_size=96, intermediate_size=160,
    num_hidden_layers=3, num_attention_heads=6, num_key_value_heads=1, head_dim=32,
    max_position_embeddings=640, rms_norm_eps=1e-5, rope_parameters={"rope_theta": 1000000.0},
    tie_word_embeddings=False)
# C: head size 48 (a step of 16 that is no power of two), 3 heads per group, odd vocabulary.
TINY_C = dict(
    architectures=["Qwen3ForCausalLM"], vocab_size=331, hidden_size=80, intermediate_size=112,
    num_hidden_layers=2, num_attention_heads=6, num_key_value_heads=2, head_dim=48,
    max_position_embeddings=400, rms_norm_eps=1e-6, rope_theta=50000.0, tie_word_embeddings=True)

# D: head size 64 and widths in multiples of 32, so that the bfloat16 mode runs on the MFMA kernels
# (attention for decode and prefill, both matrix products) inside the engine; 4 heads per group.
TINY_D = dict(
    architectures=["Qwen3ForCausalLM"], vocab_size=300, hidden_size=128, intermediate_size=192,
    num_hidden_layers=2, num_attention_heads=8, num_key_value_heads=2, head_dim=64,
    max_position_embeddings=1024, rms_norm_eps=1e-6, rope_theta=10000.0, tie_word_embeddings=False)

# E: head size 128, the size of the family's models: in bfloat16 the q|k|v product of a portion norms,
# rotates and writes the cache in its epilogue, and decode steps run the kernels the large models run.
TINY_E = dict(
    architectures=["Qwen3ForCausalLM"], vocab_size=400, hidden_size=256, intermediate_size=320,
    num_hidden_layers=2, num_attention_heads=4, num_key_value_heads=2, head_dim=128,
    max_position_embeddings=1024, rms_norm_eps=1e-6, rope_theta=1000000.0, tie_word_embeddings=False)

TINY = {"A": (TINY_A, 0, 4), "B": (TINY_B, 1, 8), "C": (TINY_C, 2, 16), "D": (TINY_D, 3, 16),
        "E": (TINY_E, 4, 16)}   # config, seed, page size


def make_folder(tmp, which: str, dtype=torch.bfloat16, norm_std=0.01, std=0.02, scale_qk=None):
    cfg_dict, seed, _ = TINY[which]
    cfg = Qwen3Config.from_dict(cfg_dict)
    folder = os.path.join(str(tmp), f"tiny_{which}_{str(dtype).split('.')[-1]}")
    write_model_folder(folder, cfg, seed, dtype=dtype, std=std, norm_std=norm_std)
    return folder
