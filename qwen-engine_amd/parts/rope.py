"""Half-split rotary position encoding.  The table is built as the reference builds
it (src/models/qwen3/model.py:75-86): 32-bit inverse frequencies 1 / theta^(2i/D),
32-bit outer product with the positions, then cos and sin, row = [cos | sin]."""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .base import Runtime, TensorInfo
from .registry import register_part


class RotaryHalf:
    fused = True   # the q/k kernel applies it from table()

    def __init__(self, spec, hidden_size: int = 0):
        self.theta = float(spec.theta)
        self.rotary_dim = int(spec.rotary_dim)
        self.max_positions = int(spec.max_positions)
        if self.rotary_dim % 2:
            raise ValueError(f"rotary_dim {self.rotary_dim} is odd")
        self._table: Optional[torch.Tensor] = None

    @staticmethod
    def expected_tensors(spec, hidden_size: int) -> Dict[str, TensorInfo]:
        return {}

    def load(self, tensors: Dict[str, torch.Tensor], rt: Runtime) -> None:
        d = self.rotary_dim
        inv_freq = 1.0 / (self.theta ** (torch.arange(0, d, 2, dtype=torch.float32) / d))
        t = torch.arange(self.max_positions, dtype=torch.float32)
        freqs = torch.outer(t, inv_freq)
        self._table = torch.cat([torch.cos(freqs), torch.sin(freqs)], dim=-1).contiguous().to(rt.device)

    def table(self) -> torch.Tensor:
        return self._table


register_part("rope_half", RotaryHalf)
