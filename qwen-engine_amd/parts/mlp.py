"""Dense gated feed-forward: down(silu(gate x) * up x), no biases
(src/models/qwen3/model.py:232-237; silu.mul as src/layers/fused_ops/silumul.py:46-53,
with the product formed in 32-bit before the one rounding).  gate and up are one
product with the two weights stacked."""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..kernels import ops
from .base import Runtime, StreamInput, TensorInfo
from .registry import register_part


class SwiGLU:
    takes_stream = True       # forward may get a StreamInput: residual sum and norm are then the gate|up product's prologue

    def __init__(self, spec, hidden_size: int):
        self.hidden = int(hidden_size)
        self.inter = int(spec.intermediate_size)
        self.w_gu = self.w_down = None
        self.interleaved = False

    @staticmethod
    def expected_tensors(spec, hidden: int) -> Dict[str, TensorInfo]:
        i = spec.intermediate_size
        return {
            "gate_proj.weight": TensorInfo((i, hidden)),
            "up_proj.weight": TensorInfo((i, hidden)),
            "down_proj.weight": TensorInfo((hidden, i)),
        }

    def load(self, tensors: Dict[str, torch.Tensor], rt: Runtime) -> None:
        g, u = tensors["gate_proj.weight"], tensors["up_proj.weight"]
        if g.dtype != u.dtype:
            g, u = g.float(), u.float()
        # gate and up rows in alternating blocks of 32, so that a product's epilogue finds the gate
        # and the up of an output side by side; widths that are no multiple of 32 keep gate | up
        self.interleaved = self.inter % 32 == 0
        self.w_gu = rt.place_matrix(ops.interleave_gate_up(g, u) if self.interleaved else torch.cat([g, u], dim=0))
        self.w_down = rt.place_matrix(tensors["down_proj.weight"])

    def forward(self, x, ctx) -> torch.Tensor:
        """Returns the feed-forward output [T, H], or float32 partial products [S, T, H] of it.
        x: the normed rows, or a StreamInput."""
        a = None
        if isinstance(x, StreamInput):
            if x.prefers_prologue(ops, self.w_gu):
                a = x.gemm(ops, self.w_gu, epilogue=ops.EPI_SILU_MUL_IL if self.interleaved else ops.EPI_SILU_MUL)
            else:
                x = x.materialize()
        if a is not None:
            pass
        elif self.interleaved and ops.gemm_silu_supported(x, self.w_gu):
            a = ops.gemm(x, self.w_gu, epilogue=ops.EPI_SILU_MUL_IL)   # silu.mul in the product's epilogue
        elif not self.interleaved and ops.gemm_fused_supported(x, self.w_gu):
            a = ops.gemm(x, self.w_gu, epilogue=ops.EPI_SILU_MUL)
        else:
            a = ops.silu_mul(ops.gemm(x, self.w_gu), interleaved=self.interleaved)
        splits = ops.gemm_branch_splits(a, self.w_down)
        if splits:   # partial products along K, added by the norm that follows
            return ops.gemm(a, self.w_down, epilogue=ops.EPI_PARTIAL, splits=splits)
        return ops.gemm(a, self.w_down)


register_part("swiglu", SwiGLU)
