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

Few rows (decode): a step is then a chain of short dependent kernels, each of which costs a few
microseconds whatever it does, so a norm and a residual sum of their own cost as much as the
products around them.  A mixer or feed-forward class may therefore say
  takes_stream = True      forward may get, instead of x, a StreamInput: the 32-bit stream, what the
                           branch before left to add to it, and the norm that stands before the
                           part; the part lets its first product do the sum and the norm
                           (StreamInput.gemm) or calls materialize()
and a norm class says with ``fusable_weight()`` (its weight and eps, or None) that it is a plain
RMSNorm that a product can take as its prologue.

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
  portion_graph_extras(tokens, device[, key]) -> dict   the same for a recorded step that is one
                                 prompt portion of ``tokens`` rows; without it, portions of a model
                                 with this part run as they come
  portion_graph_key(tokens, keys)   what of such a portion's place the part's launches depend on
                                 (keys: the keys its last row sees); the recorded step is replayed
                                 only for the same key, which portion_graph_extras gets as its third
                                 argument.  Without it nothing of the part's launches may depend on
                                 the portion's positions.
  mixed_graph_key(max_position, keys), mixed_graph_extras(rows, tokens, key, device, dynamic),
  mixed_graph_dynamic(rows, pad, tokens) with mixed_graph_dynamic_size
                                 the same for a recorded step of ``rows`` single new tokens (the step's
                                 first rows; max_position: their largest position) beside one prompt
                                 portion filled up to ``tokens`` rows: ``pad`` rows of the tables' spare
                                 row, which write nowhere, then the portion, whose last row (seeing
                                 ``keys`` keys) is the step's last.  What differs from replay to replay
                                 the part computes on the host as mixed_graph_dynamic_size integers
                                 (mixed_graph_dynamic) and finds on the device as ``dynamic`` (int32).
                                 Without these hooks such steps of a model with this part run as they come.
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


class Stream:
    """The 32-bit residual stream of a step, [T, H], with a second buffer of the same size: a
    product that adds a branch's partial products to the stream in its prologue writes the sums
    into the other buffer (its blocks read the stream while one of them writes), and the two
    change places."""

    def __init__(self, h: torch.Tensor, spare: Optional[torch.Tensor] = None):
        self.h, self.spare = h, spare

    def swap(self) -> None:
        self.h, self.spare = self.spare, self.h


@dataclass
class StreamInput:
    """The input of a part as (stream, what is still to be added to it, norm before the part)
    instead of the normed rows."""
    stream: Stream
    delta: Optional[torch.Tensor]   # None, or the branch output that the norm before the part adds to the stream
    norm: object                    # the norm part that stands before the consumer
    weight: torch.Tensor            # its weight, float32 [H]
    eps: float
    rt: "Runtime"

    @property
    def rows(self) -> int:
        return self.stream.h.shape[0]

    def fusable(self) -> bool:
        """True if a product can take the residual sum and the norm as its prologue at all: nothing to
        add, or float32 partial products and a second buffer for the sums."""
        d = self.delta
        return d is None or (d.dim() == 3 and d.dtype == torch.float32 and self.stream.spare is not None)

    def prefers_prologue(self, ops, w: torch.Tensor) -> bool:
        """True if the product against w should do the sum and the norm itself (the kernel library knows up
        to which sizes that is quicker than the norm's own kernel); else the part calls materialize()."""
        parts = 0 if self.delta is None else self.delta.shape[0]
        return self.rt.dtype == torch.bfloat16 and ops.gemm_norm_preferred(self.rows, w, parts)

    def gemm(self, ops, w: torch.Tensor, bias=None, **kw) -> torch.Tensor:
        """The product of the normed rows with w, the residual sum and the norm inside it."""
        if self.delta is None:
            return ops.gemm(self.stream.h, w, bias, norm_weight=self.weight, norm_eps=self.eps, **kw)
        y = ops.gemm(self.stream.h, w, bias, norm_weight=self.weight, norm_eps=self.eps, delta=self.delta,
                     stream_out=self.stream.spare, **kw)
        self.stream.swap()
        return y

    def materialize(self) -> torch.Tensor:
        """The normed rows as a tensor of their own (the norm's kernel, which adds delta into the stream)."""
        return self.norm.forward(self.stream.h, self.rt, delta=self.delta)


@dataclass
class CacheBinding:
    """What one schedule entry may touch of the caches in a step."""
    kv: Optional[torch.Tensor]       # [pages, 2, Hkv, P, D] of the entry whose cache is used
    group: Optional[int]             # index into ctx.block_tables / ctx.slots
    write: bool                      # False when the entry only reads another entry's cache
    state: Optional[torch.Tensor]    # [slots, *shape] fixed-size state of this entry
