"""Choice of the next token: greedy (the reference's only rule,
src/engine/executor.py:51-54: argmax, lowest index on ties) and temperature
sampling (not in the reference).

Temperature sampling draws by inverse CDF from softmax(logits / temperature) with
one uniform number per request and output position.  The number comes from a hash
of (seed, request, position), so a request's tokens do not depend on what else is
in the batch, on the order of requests or on preemption.
"""
from __future__ import annotations

import hashlib
import struct
from dataclasses import dataclass
from typing import List, Sequence

import torch

from ..kernels import ops


@dataclass
class SamplingParams:
    max_new_tokens: int = 16
    temperature: float = 0.0     # 0: greedy
    seed: int = 0
    ignore_eos: bool = False

    def validate(self) -> None:
        if self.max_new_tokens <= 0:
            raise ValueError("max_new_tokens must be positive")
        if self.temperature < 0:
            raise ValueError("temperature must not be negative")


def uniform_for(seed: int, request_key: int, position: int) -> float:
    """A number in [0, 1) with 24 random bits, fixed by (seed, request, output position)."""
    digest = hashlib.blake2b(struct.pack("<qqq", int(seed), int(request_key), int(position)),
                             digest_size=8).digest()
    return (int.from_bytes(digest, "little") >> 40) / float(1 << 24)


class Sampler:
    """Runs the sampling kernels on the logits of one step."""

    def sample(self, logits: torch.Tensor, temperatures: Sequence[float], uniforms: Sequence[float]) -> List[int]:
        """logits float32 [R, V] on the device; one temperature and one uniform per row."""
        R = logits.shape[0]
        if R == 0:
            return []
        if len(temperatures) != R or len(uniforms) != R:
            raise ValueError("one temperature and one uniform number per row are needed")
        greedy = ops.argmax(logits)
        if all(t <= 0 for t in temperatures):
            return [int(v) for v in greedy.tolist()]
        temps = torch.tensor([t if t > 0 else 1.0 for t in temperatures], dtype=torch.float32).to(logits.device)
        us = torch.tensor(list(uniforms), dtype=torch.float32).to(logits.device)
        drawn = ops.sample(logits, temps, us)
        g, d = greedy.tolist(), drawn.tolist()
        return [int(d[i]) if temperatures[i] > 0 else int(g[i]) for i in range(R)]
