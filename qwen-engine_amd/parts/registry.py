"""Registry from a spec's ``kind`` to the class that builds the part.

A part class has
  * ``expected_tensors(spec, hidden_size) -> {relative name: TensorInfo}``
  * ``__init__(spec, hidden_size)`` (no GPU needed)
  * ``load(tensors, rt)`` with the tensors named above, as stored, on the CPU
and, by role, the forward interface described in ``parts.base``.  A part whose forward
cannot be recorded into a HIP graph (it reads results back on the host, or sizes tensors
by their contents) says so with a class attribute ``graph_safe = False``.
"""
from __future__ import annotations

from typing import Dict

_PARTS: Dict[str, type] = {}


def register_part(kind: str, cls: type) -> None:
    _PARTS[kind] = cls


def unregister_part(kind: str) -> None:
    _PARTS.pop(kind, None)


def part_class(kind: str) -> type:
    try:
        return _PARTS[kind]
    except KeyError:
        raise KeyError(f"no part is registered for kind {kind!r}; known: {sorted(_PARTS)}") from None


def build_part(spec, hidden_size: int):
    return part_class(spec.kind)(spec, hidden_size)
