"""Random-weights mode: writes a model folder (config.json, model.safetensors)
from a configuration and a seed.

The reference only has the constructors' unseeded initialisation (embedding and
head N(0, 0.02), src/models/qwen3/model.py:22,367; norm weights ones, model.py:34).
Here every tensor is drawn from a generator seeded by (seed, tensor name), so a
tensor's values do not depend on which other tensors exist or on their order.
"""
from __future__ import annotations

import hashlib
import json
import os
from typing import Dict, Optional

import torch

from ..parts.model import expected_tensors


def _generator(seed: int, name: str) -> torch.Generator:
    digest = hashlib.blake2b(f"{seed}:{name}".encode(), digest_size=8).digest()
    g = torch.Generator(device="cpu")
    g.manual_seed(int.from_bytes(digest, "little") & 0x7FFFFFFFFFFFFFFF)
    return g


def random_tensors(config, seed: int, dtype: torch.dtype = torch.bfloat16, std: float = 0.02,
                   norm_std: float = 0.0, norm_dtype: Optional[torch.dtype] = None) -> Dict[str, torch.Tensor]:
    """Matrices N(0, std); norm weights 1 + N(0, norm_std); biases N(0, std).
    ``norm_dtype`` stores the norm weights in another element type than the rest."""
    spec = config.to_model_spec()
    out: Dict[str, torch.Tensor] = {}
    for name, info in expected_tensors(spec).items():
        g = _generator(seed, name)
        if info.init == "ones":
            t = torch.ones(info.shape, dtype=torch.float32)
            if norm_std:
                t = t + torch.randn(info.shape, generator=g, dtype=torch.float32) * norm_std
            out[name] = t.to(norm_dtype or dtype)
        else:
            out[name] = (torch.randn(info.shape, generator=g, dtype=torch.float32) * std).to(dtype)
    return out


def write_model_folder(folder: str, config, seed: int, dtype: torch.dtype = torch.bfloat16,
                       std: float = 0.02, norm_std: float = 0.0,
                       norm_dtype: Optional[torch.dtype] = None) -> str:
    from safetensors.torch import save_file

    os.makedirs(folder, exist_ok=True)
    d = config.to_dict()
    d["torch_dtype"] = {torch.bfloat16: "bfloat16", torch.float32: "float32"}[dtype]
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(d, f, indent=2)
    tensors = random_tensors(config, seed, dtype, std, norm_std, norm_dtype)
    save_file({k: v.contiguous() for k, v in tensors.items()}, os.path.join(folder, "model.safetensors"))
    return folder
