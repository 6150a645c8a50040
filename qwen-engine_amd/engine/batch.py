"""The flat batch that one step runs: portions of prompts beside single decoded
tokens.  The same description serves every mixer; each consumes what it needs."""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Hashable, List, Optional

import torch

from ..parts.base import Runtime


@dataclass
class SeqInfo:
    """One request's share of the step (host side)."""
    req_id: Hashable
    q_start: int        # first row of the request's tokens in the flat batch
    q_len: int          # number of its tokens in this step
    kv_before: int      # tokens already in its cache = position of its first new token
    state_slot: int
    new_request: bool   # its first step: fixed-size state starts from zero


@dataclass
class StepContext:
    rt: Runtime
    page_size: int
    num_tokens: int
    seqs: List[SeqInfo]
    token_ids: torch.Tensor            # int32 [T]
    positions: torch.Tensor            # int32 [T] absolute position of each token
    tok_seq: torch.Tensor              # int32 [T] index into seqs / rows of the block tables
    block_tables: List[torch.Tensor]   # per cache group: int32 [B, max_blocks], -1 where no page
    slots: List[torch.Tensor]          # per cache group: int32 [T] page * page_size + offset
    logit_rows: torch.Tensor           # int32 [R] rows whose logits are wanted
    state_slots: torch.Tensor          # int32 [B]
    max_position: int = 0              # largest position in the batch (host)
    # rows that are the single new token of their request, and all other rows (None: not split)
    dec_tokens: Optional[torch.Tensor] = None
    other_tokens: Optional[torch.Tensor] = None
    _tiles: dict = field(default_factory=dict)
    max_dec_position: int = 0

    def other_tiles(self, rows_per_tile: int) -> Optional[torch.Tensor]:
        """The rows of requests that bring several tokens, cut into tiles of at most
        ``rows_per_tile`` consecutive rows: int32 [tiles, 2] = (first row, rows), in groups of
        four tiles of one request (a group is filled up with tiles of 0 rows).  Built and sent
        to the device once per step and tile size."""
        if rows_per_tile <= 0:
            return None
        if rows_per_tile not in self._tiles:
            flat = prefill_tiles([(s.q_start, s.q_len) for s in self.seqs if s.q_len > 1], rows_per_tile)
            t = torch.tensor(flat, dtype=torch.int32).view(-1, 2)
            self._tiles[rows_per_tile] = t.to(self.rt.device) if flat else None
        return self._tiles[rows_per_tile]


def prefill_tiles(portions, rows_per_tile: int) -> List[int]:
    """(first row, rows) pairs, flat, for portions given as (first row, number of rows): tiles of
    at most rows_per_tile rows, in groups of four per portion, padded with (first row, 0)."""
    flat: List[int] = []
    for start, n in portions:
        tiles = [(start + r, min(rows_per_tile, n - r)) for r in range(0, n, rows_per_tile)]
        while len(tiles) % 4:
            tiles.append((start, 0))
        for t in tiles:
            flat.extend(t)
    return flat
