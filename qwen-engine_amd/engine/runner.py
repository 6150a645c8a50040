"""The step function: runs a batch of (request, its next tokens) as one batch from
the cache, and returns the logits at the wanted places.

The reference has two disjoint paths, whole prompts (src/engine/executor.py:105-168)
and one token per request (executor.py:177-208).  Here one function takes both kinds
in the same batch, cut anywhere: the attention contract is the reference's prefill
contract (tokens already cached, new tokens, keys visible up to each query's absolute
position, src/layers/fused_ops/attn.py:184-195,236-244) applied to every entry.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Hashable, List, Optional, Sequence

import torch

from ..cache.manager import CacheManager
from ..cache.plan import CachePlan
from ..config.registry import config_from_folder
from ..parts.base import CacheBinding, Runtime
from ..parts.model import DecoderModel, cache_plan, expected_tensors
from ..weights.loader import read_checked
from .batch import SeqInfo, StepContext

_TORCH_DTYPE = {"bfloat16": torch.bfloat16, "float32": torch.float32,
                "bf16": torch.bfloat16, "fp32": torch.float32}


def torch_dtype(name) -> torch.dtype:
    if isinstance(name, torch.dtype):
        return name
    try:
        return _TORCH_DTYPE[name]
    except KeyError:
        raise ValueError(f"dtype must be bfloat16 or float32, got {name!r}") from None


@dataclass
class StepEntry:
    """One request's share of a step: its next tokens, and the places among them
    (indices into ``tokens``) whose logits are wanted."""
    req_id: Hashable
    tokens: Sequence[int]
    want: Sequence[int] = field(default_factory=tuple)


def load_model(folder: str, dtype="bfloat16", device="cuda:0") -> DecoderModel:
    """Model of the architecture that config.json names, with the folder's weights."""
    config = config_from_folder(folder)
    spec = config.to_model_spec()
    model = DecoderModel(spec)
    model.config = config
    head = spec.head_name if spec.tie_head else ""
    tensors = read_checked(folder, expected_tensors(spec), tied_head_name=head)
    model.load(tensors, Runtime(device=torch.device(device), dtype=torch_dtype(dtype)))
    return model


class ModelRunner:
    """Owns the cache storage on the device and runs steps of one model."""

    def __init__(self, model: DecoderModel, page_size: int, num_pages, max_requests: int,
                 prefix_sharing: bool = False):
        if model.rt is None:
            raise RuntimeError("the model has no weights yet")
        self.model = model
        self.rt = model.rt
        self.page_size = int(page_size)
        self.plan: CachePlan = cache_plan(model.spec)
        has_state = any(s is not None for s in self.plan.entry_state)
        self.cache = CacheManager(self.plan.groups or [], num_pages, page_size, max_requests,
                                  prefix_sharing=prefix_sharing and not has_state) \
            if self.plan.groups else CacheManager([], [], page_size, max_requests)
        dev, dt = self.rt.device, self.rt.dtype
        self.kv: List[Optional[torch.Tensor]] = []
        for i, need in enumerate(self.plan.entry_kv):
            if need is None:
                self.kv.append(None)
                continue
            pages = self.cache.pools[self.plan.entry_group[i]].num_pages
            self.kv.append(torch.zeros((pages, 2, need.num_kv_heads, page_size, need.head_dim),
                                       dtype=dt, device=dev))
        self.state: List[Optional[torch.Tensor]] = []
        for need in self.plan.entry_state:
            if need is None:
                self.state.append(None)
            else:
                self.state.append(torch.zeros((max_requests, *need.shape), dtype=torch_dtype(need.dtype), device=dev))
        self.bindings = []
        for i in range(len(model.spec.schedule)):
            src = self.plan.entry_source[i]
            self.bindings.append(CacheBinding(
                kv=self.kv[src] if src is not None else None,
                group=self.plan.entry_group[i],
                write=(src == i),
                state=self.state[i]))
        self.steps_run = 0

    # ---- requests ------------------------------------------------------------------
    def add_request(self, req_id: Hashable):
        return self.cache.add_request(req_id)

    def free_request(self, req_id: Hashable) -> None:
        self.cache.free_request(req_id)

    def cache_bytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in self.kv if t is not None)

    # ---- one step ----------------------------------------------------------------------
    def build_context(self, entries: Sequence[StepEntry]) -> StepContext:
        """Reserves pages for the entries' tokens and lays the batch out flat."""
        cache, P = self.cache, self.page_size
        vocab = self.model.spec.vocab_size
        max_pos = self.model.spec.max_positions
        if not entries:
            raise ValueError("a step needs at least one entry")
        seen = set()
        for e in entries:
            if e.req_id in seen:
                raise ValueError(f"request {e.req_id!r} appears twice in one step")
            seen.add(e.req_id)
            if len(e.tokens) == 0:
                raise ValueError(f"request {e.req_id!r} brings no tokens")
            for t in e.tokens:
                if not 0 <= int(t) < vocab:
                    raise ValueError(f"token id {t} of request {e.req_id!r} is outside the vocabulary of {vocab}")
            for w in e.want:
                if not 0 <= int(w) < len(e.tokens):
                    raise ValueError(f"request {e.req_id!r} wants logits at place {w} of {len(e.tokens)} tokens")
            rc = cache.get(e.req_id)
            if rc.num_tokens + len(e.tokens) > max_pos:
                raise ValueError(f"request {e.req_id!r} would pass the model's {max_pos} positions")
        if not cache.can_reserve([(e.req_id, cache.get(e.req_id).num_tokens + len(e.tokens)) for e in entries]):
            from ..cache.manager import OutOfPages
            raise OutOfPages("the cache has too few free pages for this step")
        for e in entries:
            cache.reserve(e.req_id, cache.get(e.req_id).num_tokens + len(e.tokens))

        seqs: List[SeqInfo] = []
        token_ids: List[int] = []
        positions: List[int] = []
        tok_seq: List[int] = []
        rows: List[int] = []
        n_groups = len(cache.groups)
        slots: List[List[int]] = [[] for _ in range(n_groups)]
        q_start = 0
        for b, e in enumerate(entries):
            rc = cache.get(e.req_id)
            n = len(e.tokens)
            seqs.append(SeqInfo(e.req_id, q_start, n, rc.num_tokens, rc.state_slot, rc.new_request))
            token_ids.extend(int(t) for t in e.tokens)
            positions.extend(range(rc.num_tokens, rc.num_tokens + n))
            tok_seq.extend([b] * n)
            rows.extend(q_start + int(w) for w in e.want)
            for g in range(n_groups):
                slots[g].extend(cache.token_slots(e.req_id, g, rc.num_tokens, n))
            q_start += n
        T, B = q_start, len(entries)
        tables = []
        for g in range(n_groups):
            width = max(1, max(len(cache.block_table(e.req_id, g)) for e in entries))
            tab = [list(cache.block_table(e.req_id, g)) for e in entries]
            tables.append([row + [-1] * (width - len(row)) for row in tab])

        # one host buffer, one copy to the device
        dec_rows = [s.q_start for s in seqs if s.q_len == 1]
        other_rows = [s.q_start + i for s in seqs if s.q_len > 1 for i in range(s.q_len)]
        max_dec = max([s.kv_before for s in seqs if s.q_len == 1], default=0)
        parts = [token_ids, positions, tok_seq, rows, [s.state_slot for s in seqs], dec_rows, other_rows]
        for g in range(n_groups):
            parts.append(slots[g])
            parts.append([p for row in tables[g] for p in row])
        flat = [v for part in parts for v in part]
        host = torch.tensor(flat, dtype=torch.int32).pin_memory() if flat else torch.zeros(0, dtype=torch.int32)
        dev = host.to(self.rt.device, non_blocking=True)
        off = 0

        def take(n, shape=None):
            nonlocal off
            t = dev[off:off + n]
            off += n
            return t.view(shape) if shape is not None else t

        d_tok, d_pos, d_seq = take(T), take(T), take(T)
        d_rows, d_state = take(len(rows)), take(B)
        d_dec, d_other = take(len(dec_rows)), take(len(other_rows))
        d_slots, d_tables = [], []
        for g in range(n_groups):
            d_slots.append(take(T))
            width = len(tables[g][0])
            d_tables.append(take(B * width, (B, width)))
        return StepContext(rt=self.rt, page_size=P, num_tokens=T, seqs=seqs, token_ids=d_tok,
                           positions=d_pos, tok_seq=d_seq, block_tables=d_tables, slots=d_slots,
                           logit_rows=d_rows, state_slots=d_state, max_position=max(positions),
                           dec_tokens=d_dec, other_tokens=d_other, max_dec_position=max_dec)

    def step(self, entries: Sequence[StepEntry]) -> torch.Tensor:
        """Runs the entries' tokens as one batch; returns float32 logits [wanted, vocab] on the
        device, in the order of the entries and of their ``want``."""
        ctx = self.build_context(entries)
        for s in ctx.seqs:          # fixed-size state of a starting request begins at zero
            if s.new_request:
                for st in self.state:
                    if st is not None:
                        st[s.state_slot].zero_()
        logits = self.model.forward(ctx, self.bindings)
        for e in entries:
            self.cache.commit(e.req_id, e.tokens)
        self.steps_run += 1
        return logits
