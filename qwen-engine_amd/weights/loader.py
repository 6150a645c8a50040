"""Weights from a model folder, by tensor name.

The reference reads every ``*.safetensors`` file of the folder and copies tensors
into parameters of the same name, recording what did not fit without ever raising
(src/models/qwen3/utils.py:67-103).  Here the folder is checked against the tensors
the model expects before anything is placed: missing names, unexpected names and
wrong shapes are reported together in one error.
"""
from __future__ import annotations

import os
from collections.abc import Mapping
from typing import Dict, Iterator, List, Tuple

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


class LazyTensors(Mapping):
    """The checked tensors of a model folder by name; a tensor is read from its file when it is
    asked for, as stored, onto the CPU, and nothing of it is kept here.  The model asks part by
    part, so that the host never holds more than one part's tensors (the reference reads every
    tensor of the checkpoint into one dict first, src/models/qwen3/utils.py:77-82)."""

    def __init__(self, handles, where: Dict[str, int], names: Dict[str, str]):
        self._handles, self._where, self._names = handles, where, names   # names: name here -> name in the files

    def __getitem__(self, name: str) -> torch.Tensor:
        real = self._names[name]
        return self._handles[self._where[real]].get_tensor(real)

    def __iter__(self) -> Iterator[str]:
        return iter(self._names)

    def __contains__(self, name) -> bool:       # (asking whether a tensor is there reads nothing)
        return name in self._names

    def __len__(self) -> int:
        return len(self._names)

    def subset(self, prefix: str) -> "LazyTensors":
        """The tensors whose names begin with ``prefix``, under their names without it."""
        return LazyTensors(self._handles, self._where,
                           {k[len(prefix):]: real for k, real in self._names.items() if k.startswith(prefix)})


def read_checked(folder: str, expected: Dict[str, TensorInfo], tied_head_name: str = "") -> LazyTensors:
    """Checks the folder's safetensors headers against the expected tensors and returns them as a
    mapping that reads each tensor when it is asked for (as stored, on the CPU).

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
    return LazyTensors(handles, where, {name: name for name in expected})
