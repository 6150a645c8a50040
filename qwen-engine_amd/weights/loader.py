"""Weights from a model folder, by tensor name.

The reference reads every ``*.safetensors`` file of the folder and copies tensors
into parameters of the same name, recording what did not fit without ever raising
(src/models/qwen3/utils.py:67-103).  Here the folder is checked against the tensors
the model expects before anything is placed: missing names, unexpected names and
wrong shapes are reported together in one error.
"""
from __future__ import annotations

import os
from typing import Dict, List, Tuple

import torch

from ..parts.base import TensorInfo


class WeightError(ValueError):
    """The model folder does not hold the tensors the model expects."""

    def __init__(self, folder: str, missing: List[str], unexpected: List[str],
                 wrong_shape: List[Tuple[str, Tuple[int, ...], Tuple[int, ...]]]):
        self.missing, self.unexpected, self.wrong_shape = missing, unexpected, wrong_shape
        lines = [f"the weights in {folder} do not fit the model:"]
        if missing:
            lines.append(f"  missing tensors ({len(missing)}): " + ", ".join(missing))
        if unexpected:
            lines.append(f"  unexpected tensors ({len(unexpected)}): " + ", ".join(unexpected))
        if wrong_shape:
            lines.append(f"  wrong shapes ({len(wrong_shape)}): " + ", ".join(
                f"{n} is {list(got)}, expected {list(want)}" for n, got, want in wrong_shape))
        super().__init__("\n".join(lines))


def safetensors_files(folder: str) -> List[str]:
    if not os.path.isdir(folder):
        raise ValueError(f"model folder not found: {folder}")
    files = sorted(f for f in os.listdir(folder) if f.endswith(".safetensors"))
    if not files:
        raise ValueError(f"no .safetensors files found in {folder}")   # utils.py:74-75
    return [os.path.join(folder, f) for f in files]


def read_checked(folder: str, expected: Dict[str, TensorInfo], tied_head_name: str = "") -> Dict[str, torch.Tensor]:
    """All expected tensors of the folder, as stored, on the CPU.

    ``tied_head_name``: a tensor of this name is tolerated though not expected (a
    checkpoint with tied embeddings may store the head again); it is not read.
    """
    from safetensors import safe_open

    handles = []
    where: Dict[str, int] = {}
    shapes: Dict[str, Tuple[int, ...]] = {}
    for path in safetensors_files(folder):
        f = safe_open(path, framework="pt", device="cpu")
        handles.append(f)
        for name in f.keys():
            where[name] = len(handles) - 1
            shapes[name] = tuple(f.get_slice(name).get_shape())
    missing = sorted(n for n in expected if n not in where)
    unexpected = sorted(n for n in where if n not in expected and n != tied_head_name)
    wrong = sorted((n, shapes[n], tuple(expected[n].shape)) for n in expected
                   if n in where and shapes[n] != tuple(expected[n].shape))
    if missing or unexpected or wrong:
        raise WeightError(folder, missing, unexpected, wrong)
    return {name: handles[where[name]].get_tensor(name) for name in expected}
