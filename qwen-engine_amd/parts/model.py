"""The decoder: embedding, the layers in the order of the schedule, final norm on
the wanted rows, head (src/models/qwen3/model.py:349-359,420-422; the head is applied
only where logits are asked for, and gives 32-bit logits)."""
from __future__ import annotations

from typing import Dict, List, Optional, Tuple

import torch

from ..cache.plan import CachePlan, plan_cache
from ..config.spec import ModelSpec
from ..kernels import ops
from .base import CacheBinding, Runtime, Stream, TensorInfo, sub_tensors
from .registry import build_part, part_class


def expected_tensors(spec: ModelSpec) -> Dict[str, TensorInfo]:
    """Every tensor the model folder must hold, by checkpoint name."""
    out: Dict[str, TensorInfo] = {spec.embed_name: TensorInfo((spec.vocab_size, spec.hidden_size), "normal", "matrix")}
    for layer in spec.layers:
        for rel, info in part_class(layer.kind).expected_tensors(layer, spec.hidden_size).items():
            out[f"{layer.prefix}.{rel}"] = info
    norm_rel = part_class(spec.final_norm.kind).expected_tensors(spec.final_norm, spec.hidden_size)
    base = spec.final_norm_name[:-len(".weight")] if spec.final_norm_name.endswith(".weight") else spec.final_norm_name
    for rel, info in norm_rel.items():
        out[f"{base}.{rel}"] = info
    if not spec.tie_head:
        out[spec.head_name] = TensorInfo((spec.vocab_size, spec.hidden_size), "normal", "matrix")
    for extra in (spec.stream_prologue, spec.logit_epilogue):
        if extra is not None:
            for rel, info in part_class(extra.kind).expected_tensors(extra, spec.hidden_size).items():
                out[_join(getattr(extra, "prefix", ""), rel)] = info
    return out


def _join(prefix: str, rel: str) -> str:
    return f"{prefix}.{rel}" if prefix else rel


def cache_plan(spec: ModelSpec) -> CachePlan:
    """Every block kind says itself what its parts keep per request (``cache_needs(spec, hidden)``: a list
    of (keys and values, fixed-size state), one per cache user of the block; none if it has no such method)."""
    needs = []
    for entry in spec.schedule:
        layer = spec.layers[entry.layer]
        cls = part_class(layer.kind)
        users = list(cls.cache_needs(layer, spec.hidden_size)) if hasattr(cls, "cache_needs") else []
        needs.append((users, entry.cache_from))
    return plan_cache(needs)


class DecoderModel:
    def __init__(self, spec: ModelSpec):
        spec.validate()
        self.spec = spec
        self.blocks = [build_part(layer, spec.hidden_size) for layer in spec.layers]
        self.final_norm = build_part(spec.final_norm, spec.hidden_size)
        # optional parts around the layers: one that changes the stream right after the embedding
        # (forward(h, ctx), in place), one that changes the logits after the head (forward(logits, ctx))
        self.prologue = build_part(spec.stream_prologue, spec.hidden_size) if spec.stream_prologue is not None else None
        self.epilogue = build_part(spec.logit_epilogue, spec.hidden_size) if spec.logit_epilogue is not None else None
        self.embed: Optional[torch.Tensor] = None
        self.head: Optional[torch.Tensor] = None
        self.rt: Optional[Runtime] = None

    @property
    def graph_safe(self) -> bool:
        """A part whose forward reads results back on the host, sizes tensors by their contents or
        walks the requests of a step sets ``graph_safe = False``; the decode steps of a model with
        such a part are run as they come instead of being recorded once and replayed."""
        return all(getattr(p, "graph_safe", True) for p in (*self.blocks, *self._around()))

    def _around(self):
        return [p for p in (self.final_norm, self.prologue, self.epilogue) if p is not None]

    def all_parts(self):
        """Every part of the model, the parts inside the blocks included."""
        for b in self.blocks:
            yield b
            yield from (b.parts() if hasattr(b, "parts") else ())
        yield from self._around()

    def load(self, tensors: Dict[str, torch.Tensor], rt: Runtime) -> None:
        spec = self.spec
        self.rt = rt
        self.embed = rt.place_matrix(tensors[spec.embed_name])
        for layer, block in zip(spec.layers, self.blocks):
            block.load(sub_tensors(tensors, layer.prefix + "."), rt)
        base = spec.final_norm_name[:-len(".weight")] if spec.final_norm_name.endswith(".weight") else spec.final_norm_name
        self.final_norm.load(sub_tensors(tensors, base + "."), rt)
        self.head = self.embed if spec.tie_head else rt.place_matrix(tensors[spec.head_name])
        for part, part_spec in ((self.prologue, spec.stream_prologue), (self.epilogue, spec.logit_epilogue)):
            if part is not None:
                pre = getattr(part_spec, "prefix", "")
                pre = pre + "." if pre else ""
                names = part_class(part_spec.kind).expected_tensors(part_spec, spec.hidden_size)
                part.load({rel: tensors[pre + rel] for rel in names}, rt)

    def weight_bytes_read_per_step(self) -> int:
        """Bytes of every weight a step uses once: all tensors that the parts hold (the parts inside the
        parts included), a layer that the schedule runs n times n times; the embedding table only where
        it is the head.  Tables that a step reads a few rows of (a position encoding's) are the parts'
        to leave out: they keep them under a name that begins with an underscore."""
        seen = set()

        def held(part) -> int:
            total = 0
            for name, v in vars(part).items():
                if name.startswith("_"):
                    continue
                if isinstance(v, torch.Tensor):
                    if v.data_ptr() not in seen:
                        seen.add(v.data_ptr())
                        total += v.numel() * v.element_size()
                elif hasattr(v, "load") and hasattr(v, "expected_tensors"):     # a part inside the part
                    total += held(v)
            return total

        counts: Dict[int, int] = {}
        for e in self.spec.schedule:
            counts[e.layer] = counts.get(e.layer, 0) + 1
        total = 0
        for idx, n in counts.items():
            total += n * held(self.blocks[idx])
        for part in self._around():
            total += held(part)
        if self.head is not None and self.head.data_ptr() not in seen:
            total += self.head.numel() * self.head.element_size()
        return total

    def forward(self, ctx, bindings: List[CacheBinding]) -> torch.Tensor:
        """Runs the tokens of ctx through the schedule; returns float32 logits [R, V]."""
        with ops.one_stream():           # (the whole step runs on the stream that is current now)
            h = ops.embedding(ctx.token_ids, self.embed)
            if self.prologue is not None:
                self.prologue.forward(h, ctx)
            # (few rows: a second buffer, so that a product can do the residual sum before it, see Stream)
            stream = Stream(h, torch.empty_like(h) if h.shape[0] <= ops.gemm_norm_max_rows() else None)
            pending = None
            for i, entry in enumerate(self.spec.schedule):
                pending = self.blocks[entry.layer].forward(stream, pending, ctx, bindings[i])   # (the entry's users' bindings)
            h = stream.h
            R = ctx.logit_rows.shape[0]
            if R == 0:
                return torch.empty((0, self.spec.vocab_size), dtype=torch.float32, device=h.device)
            x = self.final_norm.forward(h, ctx.rt, delta=pending, rows=ctx.logit_rows)
            logits = ops.gemm(x, self.head, out_dtype=torch.float32)
            if self.epilogue is not None:
                logits = self.epilogue.forward(logits, ctx)
            return logits
