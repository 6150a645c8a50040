"""Interfaces of the parts a layer is put together from.  No part knows which
model it is in: each gets its sizes and constants from its spec.

Norm          forward(h, rt, delta=None, rows=None) -> x
              h is the 32-bit residual stream [T, H]; with ``delta`` (a branch output, see
              below) the sum h + delta is normed and written back to h; with ``rows`` only
              those rows are normed.
Mixer         forward(x, ctx, binding) -> y      x, y [T, H] in the activation type
              cache_need(spec) -> KVNeed | None, state_need(spec, hidden) -> StateNeed | None
FeedForward   forward(x, ctx) -> y
              A mixer's or feed-forward's y is [T, H] in the activation type, or float32 [S, T, H]:
              partial products whose sum over S, taken in order, is the output (the norm adds them).
Position      table() for the fused kernel, or apply(packed, positions, num_q, num_k) in place
              on a [T, Hq + 2 Hkv, D] tensor of q | k | v heads.
Stream prologue   forward(h, ctx) -> None: changes the 32-bit stream in place right after the
              embedding (a scale, an added table of positions).
Logit epilogue    forward(logits, ctx) -> logits on the float32 logits [R, V] (a scale, a soft cap).

What a part needs prepared per step beyond the flat batch, it asks for itself; the step function
knows none of it.  A part class may define (all optional, all static):
  step_extras(seqs) -> dict      from the step's SeqInfo list, on the host: int32 numpy arrays (sent
                                 to the device with the batch, in the one copy) and plain numbers;
                                 the part finds them as ctx.extras[its class]
  graph_key(max_position)        what of a decode step's positions the part's launches depend on
                                 (a recorded step is replayed only for the same key)
  graph_extras(rows, key, device) -> dict   the same entries as step_extras for a recorded step of
                                 ``rows`` single new tokens whose positions give ``key``, as
                                 tensors that stay as they are for every replay
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, NamedTuple, Optional, Tuple

import torch


class TensorInfo(NamedTuple):
    shape: Tuple[int, ...]
    init: str = "normal"   # "normal": N(0, std); "ones": norm weight; "zeros": bias
    role: str = "matrix"   # "matrix" keeps the stored element type in bfloat16 mode; "vector" is held in 32-bit


def sub_tensors(tensors, prefix: str):
    """The tensors whose names begin with ``prefix``, under their names without it.  A mapping
    that reads tensors on demand (it has ``subset``) stays one: nothing is read here."""
    if hasattr(tensors, "subset"):
        return tensors.subset(prefix)
    return {k[len(prefix):]: v for k, v in tensors.items() if k.startswith(prefix)}


@dataclass
class Runtime:
    """Where and in which element type the engine computes."""
    device: torch.device
    dtype: torch.dtype   # activations and cache: torch.bfloat16 or torch.float32

    def place_matrix(self, t: torch.Tensor) -> torch.Tensor:
        """Matrices and tables: bfloat16 stays bfloat16, a tensor stored in 32-bit stays
        so, integers become int32; in float32 mode every float becomes float32."""
        if t.dtype in (torch.int8, torch.int16, torch.int32, torch.int64, torch.uint8):
            return t.to(torch.int32).contiguous().to(self.device)
        if self.dtype == torch.float32 or t.dtype == torch.float32:
            return t.to(torch.float32).contiguous().to(self.device)
        return t.to(torch.bfloat16).contiguous().to(self.device)

    def place_vector(self, t: torch.Tensor) -> torch.Tensor:
        """Norm weights and biases enter 32-bit arithmetic only: held in float32 (exact)."""
        return t.to(torch.float32).contiguous().to(self.device)


@dataclass
class CacheBinding:
    """What one schedule entry may touch of the caches in a step."""
    kv: Optional[torch.Tensor]       # [pages, 2, Hkv, P, D] of the entry whose cache is used
    group: Optional[int]             # index into ctx.block_tables / ctx.slots
    write: bool                      # False when the entry only reads another entry's cache
    state: Optional[torch.Tensor]    # [slots, *shape] fixed-size state of this entry
