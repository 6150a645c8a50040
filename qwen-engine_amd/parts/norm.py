"""RMSNorm over the 32-bit residual stream, with the residual sum fused in.
Formula: src/layers/ops/layernorm.py:50-89 (all three factors in 32-bit, one rounding)."""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..kernels import ops
from .base import Runtime, TensorInfo
from .registry import register_part


class RMSNorm:
    def __init__(self, spec, size: int):
        self.eps = float(spec.eps)
        self.size = int(size)
        self.weight: Optional[torch.Tensor] = None

    @staticmethod
    def expected_tensors(spec, size: int) -> Dict[str, TensorInfo]:
        return {"weight": TensorInfo((size,), "ones", "vector")}

    def load(self, tensors: Dict[str, torch.Tensor], rt: Runtime) -> None:
        self.weight = rt.place_vector(tensors["weight"])

    def fusable_weight(self):
        """(weight, eps): this is a plain RMSNorm, which a product can take as its prologue."""
        return self.weight, self.eps

    def forward(self, h: torch.Tensor, rt: Runtime, delta: Optional[torch.Tensor] = None,
                rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        return ops.rmsnorm(h, self.weight, self.eps, rt.dtype, delta=delta, rows=rows)


register_part("rmsnorm", RMSNorm)
