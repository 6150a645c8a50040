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
    scatter_pages: bool = True       # a fresh pool hands its pages out in a scattered order (see cache.manager.PagePool)
    seed: int = 0
    debug_poison: bool = False       # NaN into every cache page when it is handed out and when it goes back
    record_mixed_steps: bool = True  # steps of single new tokens beside one prompt portion are replayed from recorded graphs
    graph_record_after: int = 2      # a step with prompt tokens is recorded when its shape is met for this many times
    graph_memory_bytes: int = 8 << 30  # recorded steps may hold this much device memory; the least recently used go first
    # num_blocks None and this set: the pool takes this fraction of the device memory that is free once
    # the weights are loaded, less graph_memory_bytes (the reference has the fixed formula only, main.py:23)
    gpu_memory_fraction: Optional[float] = None

    def pages_per_group(self, free_bytes: Optional[int] = None, bytes_per_page: int = 0) -> int:
        """Pages of every cache group.  ``free_bytes`` (device memory free after the weights) and
        ``bytes_per_page`` (a page of every layer of all groups together) are asked for only with
        gpu_memory_fraction: all groups get the same number of pages, what fits into the fraction."""
        if self.num_blocks is not None:
            return self.num_blocks
        per_seq = (self.max_model_len + self.block_size - 1) // self.block_size
        if self.gpu_memory_fraction is not None:
            if free_bytes is None or bytes_per_page <= 0:
                raise ValueError("gpu_memory_fraction needs the free device memory and the bytes of a page")
            pages = int((free_bytes * self.gpu_memory_fraction - self.graph_memory_bytes) // bytes_per_page)
            if pages < per_seq:
                raise ValueError(f"{self.gpu_memory_fraction:.2f} of {free_bytes >> 20} MiB free, less "
                                 f"{self.graph_memory_bytes >> 20} MiB for recorded steps, holds {max(pages, 0)} pages "
                                 f"of {bytes_per_page} bytes: fewer than the {per_seq} of one request of max_model_len")
            return pages
        return self.max_num_seqs * per_seq  # main.py:23

    def validate(self) -> None:
        if self.dtype not in ("bfloat16", "float32"):
            raise ValueError(f"dtype must be bfloat16 or float32, got {self.dtype!r}")
        for k in ("block_size", "max_num_seqs", "max_model_len", "max_step_tokens", "prefill_chunk"):
            if getattr(self, k) <= 0:
                raise ValueError(f"{k} must be positive")
        if self.num_blocks is not None and self.num_blocks <= 0:
            raise ValueError("num_blocks must be positive")
        if self.gpu_memory_fraction is not None and not 0.0 < self.gpu_memory_fraction <= 1.0:
            raise ValueError("gpu_memory_fraction must lie in (0, 1]")
        if self.graph_record_after <= 0 or self.graph_memory_bytes < 0:
            raise ValueError("graph_record_after must be positive and graph_memory_bytes not negative")
