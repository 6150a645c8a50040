"""A pre-norm residual block: x += mixer(norm(x)); x += ffn(norm(x))
(src/models/qwen3/model.py:278-298).  The residual stream is kept in 32-bit and each
residual sum is fused into the norm that follows it, so the block hands its last
branch output on as ``pending`` instead of adding it itself."""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .base import CacheBinding, Runtime, Stream, StreamInput, TensorInfo, sub_tensors
from ..kernels import ops
from .registry import build_part, part_class, register_part

def _names(spec):
    """Checkpoint names of the four parts inside the layer's prefix (LayerSpec.part_names)."""
    return spec.part_names


class PreNormBlock:
    def __init__(self, spec, hidden_size: int):
        self.spec = spec
        self.hidden = int(hidden_size)
        self.mixer_norm = build_part(spec.mixer_norm, hidden_size)
        self.mixer = build_part(spec.mixer, hidden_size)
        self.ffn_norm = build_part(spec.ffn_norm, hidden_size)
        self.ffn = build_part(spec.ffn, hidden_size)

    @property
    def graph_safe(self) -> bool:
        """False if any part of the block says that its forward cannot be recorded into a graph."""
        return all(getattr(p, "graph_safe", True) for p in (self.mixer_norm, self.mixer, self.ffn_norm, self.ffn))

    @property
    def graph_safe_with_state(self) -> bool:
        """A part with per-request state is recorded into graphs only if it says itself that it can be."""
        return getattr(self.mixer, "graph_safe", False) is True

    def parts(self):
        return (self.mixer_norm, self.mixer, self.ffn_norm, self.ffn)

    @staticmethod
    def cache_needs(spec, hidden: int):
        """What the block's parts keep per request, one (keys and values, fixed-size state) per cache
        user, in the order in which forward gets their bindings: this block has one, its mixer."""
        cls = part_class(spec.mixer.kind)
        kv = cls.cache_need(spec.mixer) if hasattr(cls, "cache_need") else None
        state = cls.state_need(spec.mixer, hidden) if hasattr(cls, "state_need") else None
        return [(kv, state)]

    @staticmethod
    def expected_tensors(spec, hidden: int) -> Dict[str, TensorInfo]:
        out: Dict[str, TensorInfo] = {}
        for name, sub in zip(_names(spec), (spec.mixer_norm, spec.mixer, spec.ffn_norm, spec.ffn)):
            for rel, info in part_class(sub.kind).expected_tensors(sub, hidden).items():
                out[f"{name}.{rel}"] = info
        return out

    def load(self, tensors: Dict[str, torch.Tensor], rt: Runtime) -> None:
        for name, part in zip(_names(self.spec), (self.mixer_norm, self.mixer, self.ffn_norm, self.ffn)):
            part.load(sub_tensors(tensors, name + "."), rt)

    def forward(self, h, pending: Optional[torch.Tensor], ctx, bindings) -> torch.Tensor:
        """h: the 32-bit residual stream, a tensor (updated in place) or a Stream (whose buffers may
        change places).  pending: branch output not yet added to the stream, or None.  bindings: one
        CacheBinding per cache user of the block (cache_needs), here the mixer's.  Returns the
        feed-forward output, to be added by whoever norms next.  A branch output is [T, H] in the
        activation type, or float32 [S, T, H]: partial products that the norm adds in the order of S."""
        stream = h if isinstance(h, Stream) else Stream(h)
        x = self._input(self.mixer_norm, self.mixer, stream, pending, ctx)
        a = self.mixer.forward(x, ctx, bindings[0])
        x = self._input(self.ffn_norm, self.ffn, stream, a, ctx)
        return self.ffn.forward(x, ctx)

    @staticmethod
    def _input(norm, part, stream: Stream, delta, ctx):
        """The part's input: the normed rows, or, with few rows (the model then gave the stream a second
        buffer) and where both the norm and the part can do it, the stream, what is to be added, and
        the norm, for the part's first product."""
        if (getattr(part, "takes_stream", False) and hasattr(norm, "fusable_weight") and
                stream.spare is not None):
            fw = norm.fusable_weight()
            si = StreamInput(stream, delta, norm, fw[0], fw[1], ctx.rt) if fw is not None else None
            if si is not None and si.fusable():
                return si
        return norm.forward(stream.h, ctx.rt, delta=delta)


register_part("prenorm_block", PreNormBlock)
