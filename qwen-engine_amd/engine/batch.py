"""The flat batch that one step runs: portions of prompts beside single decoded
tokens.  The same description serves every mixer; each consumes what it needs."""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, Hashable, List, Optional

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
    # int32, an entry per row of the block tables, or None: how many of the request's first keys lie in
    # pages that other requests read as well (a shared prefix).  A hint for kernels that choose between
    # loads that leave a line in the caches and loads that stream past them; no result depends on it.
    shared_keys: Optional[torch.Tensor] = None
    # What single parts asked to have prepared for this step, by part class (see
    # ``parts.base``: step_extras / graph_extras), and a place where a part may keep what it
    # builds once per step and shares between its layers.
    extras: Dict[type, dict] = field(default_factory=dict)
    memo: dict = field(default_factory=dict)
