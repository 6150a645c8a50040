"""Run-time sizes of the engine.  The names follow the constants of the
reference's main.py:19-27 (max_num_seqs, max_model_len, block_size, num_blocks);
the token budget and the prompt portion size have no counterpart there."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional


@dataclass
class EngineConfig:
    dtype: str = "bfloat16"          # "bfloat16" or "float32"
    block_size: int = 16             # tokens in a page of the cache
    num_blocks: Optional[int] = None  # pages per cache group; None: from max_num_seqs * max_model_len
    max_num_seqs: int = 4            # requests that run at a time
    max_model_len: int = 256         # prompt + generated tokens of one request
    max_step_tokens: int = 2048      # token budget of one step
    prefill_chunk: int = 512         # largest portion of one prompt in a step in which some request decodes
    enable_prefix_sharing: bool = True
    keep_freed_prefixes: bool = True   # shared pages of finished requests stay until their memory is needed
    seed: int = 0
    debug_poison: bool = False       # NaN into every cache page when it is handed out and when it goes back

    def pages_per_group(self) -> int:
        if self.num_blocks is not None:
            return self.num_blocks
        per_seq = (self.max_model_len + self.block_size - 1) // self.block_size
        return self.max_num_seqs * per_seq  # main.py:23

    def validate(self) -> None:
        if self.dtype not in ("bfloat16", "float32"):
            raise ValueError(f"dtype must be bfloat16 or float32, got {self.dtype!r}")
        for k in ("block_size", "max_num_seqs", "max_model_len", "max_step_tokens", "prefill_chunk"):
            if getattr(self, k) <= 0:
                raise ValueError(f"{k} must be positive")
        if self.num_blocks is not None and self.num_blocks <= 0:
            raise ValueError("num_blocks must be positive")
