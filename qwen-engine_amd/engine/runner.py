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

import numpy as np
import torch

from ..cache.manager import CacheManager, OutOfPages
from ..cache.plan import CachePlan
from ..config.registry import config_from_folder
from ..kernels import ops
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
    """Owns the cache storage on the device and runs steps of one model.

    The block tables live on the device, one row per state slot; a step uploads only the
    entries that changed (new pages, pages a window has passed) together with the batch's
    tokens, positions and cache slots in one copy.  Steps in which every request brings one
    token and wants its logits (decoding) are recorded once per batch size as a HIP graph
    and replayed, so that their launch cost does not grow with the number of kernels.
    """

    # A step that is one prompt portion of a round length (a whole number of PORTION_GRAPH_STEP tokens,
    # at least PORTION_GRAPH_MIN) is recorded once per length too: a portion is a few hundred kernels
    # of some microseconds each, which the host cannot launch as fast as the device runs them.
    PORTION_GRAPH_MIN = 256
    PORTION_GRAPH_STEP = 128
    # A step of single new tokens beside exactly one prompt portion (what a server runs while requests
    # keep arriving) is recorded too: the single tokens' rows are filled up as in a decode graph, the
    # portion to a multiple of MIXED_GRAPH_STEP tokens with rows of the tables' spare row that write
    # nowhere.  Run as it comes, such a step costs the host some 370 launches (3.7 ms at the small
    # model's sizes, more than its kernels take).
    MIXED_GRAPH_STEP = 128
    MIXED_GRAPH_MAX_TOKENS = 2048
    # Recorded graphs kept; the least recently used goes first.  Each holds its own activations and
    # workspaces (tens of MB at the small model's sizes, a GB for a long portion at the large models'),
    # so they are bounded by their bytes too (graph_memory_bytes).  A server whose batch
    # and contexts wander passes through 15 row counts up to 64 rows times a bucket per 1024 keys, and
    # recording a step again costs several replays of it.
    MAX_GRAPHS = 96

    def __init__(self, model: DecoderModel, page_size: int, num_pages, max_requests: int,
                 prefix_sharing: bool = False, use_graphs: Optional[bool] = None,
                 keep_freed_prefixes: bool = False, debug_poison: bool = False,
                 record_mixed_steps: bool = True, graph_record_after: int = 1,
                 graph_memory_bytes: int = 8 << 30, scatter_pages: bool = True):
        if model.rt is None:
            raise RuntimeError("the model has no weights yet")
        self.model = model
        self.rt = model.rt
        self.page_size = int(page_size)
        self.max_requests = int(max_requests)
        self.plan: CachePlan = cache_plan(model.spec)
        has_state = any(s is not None for s in self.plan.user_state)
        self.cache = CacheManager(self.plan.groups or [], num_pages, page_size, max_requests,
                                  prefix_sharing=prefix_sharing and not has_state,
                                  keep_freed_prefixes=keep_freed_prefixes, scatter_pages=scatter_pages) \
            if self.plan.groups else CacheManager([], [], page_size, max_requests)
        dev, dt = self.rt.device, self.rt.dtype
        # debug_poison: the storage starts as NaN, and every page is filled with NaN again when it
        # is handed out and when it goes back, so that a read of a key that was never written, or of
        # a page that is no longer the request's, makes the logits NaN instead of slightly wrong
        self.debug_poison = bool(debug_poison)
        self.cache.track_pages = self.debug_poison
        self.pages_poisoned = 0
        self.kv: List[Optional[torch.Tensor]] = []
        for u, need in enumerate(self.plan.user_kv):         # (per cache user of the schedule, see CachePlan)
            if need is None:
                self.kv.append(None)
                continue
            pages = self.cache.pools[self.plan.user_group[u]].num_pages
            self.kv.append(torch.full((pages, 2, need.num_kv_heads, page_size, need.head_dim),
                                      float("nan") if self.debug_poison else 0.0, dtype=dt, device=dev))
        self.state: List[Optional[torch.Tensor]] = []
        for need in self.plan.user_state:
            if need is None:
                self.state.append(None)
            else:
                # (one slot more than requests: the spare one belongs to the rows that fill a graph up)
                self.state.append(torch.zeros((max_requests + 1, *need.shape), dtype=torch_dtype(need.dtype), device=dev))
        # per schedule entry: one binding per cache user of its block, in the block's order
        self.bindings = []
        for users in self.plan.entry_users:
            row = []
            for u in users:
                src = self.plan.user_source[u]
                row.append(CacheBinding(
                    kv=self.kv[src] if src is not None else None,
                    group=self.plan.user_group[u],
                    write=(src == u),
                    state=self.state[u]))
            self.bindings.append(row)
        # device copies of the block tables: [state slots, pages a request can hold]
        per_request = (model.spec.max_positions + page_size - 1) // page_size
        # (a table is indexed by position // page size: with a window the indices go on growing
        # while the entries behind the window are -1, so only a group that keeps all keys is
        # bounded by its pool)
        self.table_width = [max(1, per_request if grp.window is not None else min(pool.num_pages, per_request))
                            for grp, pool in zip(self.cache.groups, self.cache.pools)]
        # one row more than there are state slots: the spare row's entries always name page 0
        # of their pool.  It is the table row of the rows that fill a recorded decode graph up and of
        # the stand-in batch while recording: they stand at position 0 and write nowhere, and what
        # they read there lies inside the storage whatever the live requests hold.
        self.tables = [torch.full((max_requests + 1, w), -1, dtype=torch.int32, device=dev) for w in self.table_width]
        for t in self.tables:
            t[max_requests].zero_()            # (every entry: the stand-in of a recorded prompt portion reads them all)
        self.spare_row = max_requests
        # per table row: the request's first keys that other requests read too (StepContext.shared_keys)
        self.shared_keys = torch.zeros(max_requests + 1, dtype=torch.int32, device=dev)
        self._shared_keys_host = [0] * (max_requests + 1)
        # positions that a row standing on the spare row may have: inside every group's table row, and the model's
        self._spare_positions = min([w * page_size for w in self.table_width] + [model.spec.max_positions])
        # a part with per-request state is recorded into graphs only if it says that it can be
        # (``graph_safe = True`` on the class); any other part unless it says that it cannot
        stateful_ok = all(all(self.plan.user_state[u] is None for u in users) or
                          getattr(model.blocks[e.layer], "graph_safe_with_state", False) is True
                          for users, e in zip(self.plan.entry_users, model.spec.schedule))
        graph_safe = stateful_ok and getattr(model, "graph_safe", True)
        self.use_graphs = (dt == torch.bfloat16 and graph_safe) if use_graphs is None else bool(use_graphs)
        # the part classes that want something prepared for every step (parts.base: step_extras)
        self._step_classes = []
        for part in model.all_parts():
            cls = type(part)
            if hasattr(cls, "step_extras") and cls not in self._step_classes:
                self._step_classes.append(cls)
        self._graphs = {}
        # portions are recorded only if every part that wants something prepared can say what a
        # recorded portion needs (parts.base: portion_graph_extras)
        self._portion_graphs = all(hasattr(cls, "portion_graph_extras") for cls in self._step_classes)
        # ... and mixed steps only if they can say the same for those, and no part keeps state of its own
        self._mixed_graphs = (all(hasattr(cls, "mixed_graph_extras") for cls in self._step_classes) and not has_state
                              and bool(record_mixed_steps))
        # A step of prompt tokens (a portion, or a portion beside single tokens) is recorded only when its
        # shape has been met this many times: recording costs two runs of the step, a capture and three
        # waits for the device, which a shape that never comes back does not earn.  Decode steps are
        # recorded at once (their shapes are few and come back every step).
        self.graph_record_after = max(1, int(graph_record_after))
        self.graph_memory_bytes = int(graph_memory_bytes)
        self._graph_seen = {}
        self.graph_misses = 0                      # steps of a shape that is recorded, run as they came because it was not yet
        self._stage: Optional[torch.Tensor] = None     # pinned host buffer of a step's integer arrays
        self._stage_np = None
        self._stage_event = torch.cuda.Event()
        self.steps_run = 0
        self.graph_steps = 0                       # steps replayed from a recorded graph, and by what they were:
        self.graph_steps_of = {"decode": 0, "portion": 0, "mixed": 0}
        self.graphs_recorded = 0

    @staticmethod
    def graph_rows(n: int) -> int:
        """The rows of the recorded decode graph that a batch of n single tokens replays: n itself up
        to 8, the next multiple of 8 up to 64, of 32 beyond."""
        if n <= 8:
            return n
        step = 8 if n <= 64 else 32
        return -(-n // step) * step

    def _graph_for(self, key, kind: str, record):
        """The recorded step for ``key`` (most recently used last), recorded now by ``record()`` if its
        shape has been met often enough, or None: the step then runs as it comes."""
        rec = self._graphs.pop(key, None)
        if rec is None:
            if kind != "decode":
                seen = self._graph_seen.get(key, 0) + 1
                if seen < self.graph_record_after:
                    if len(self._graph_seen) >= 4096:          # (shapes that never came back)
                        self._graph_seen.clear()
                    self._graph_seen[key] = seen
                    self.graph_misses += 1
                    return None
                self._graph_seen.pop(key, None)
            before = torch.cuda.memory_allocated(self.rt.device)
            rec = record()
            rec["bytes"] = max(0, torch.cuda.memory_allocated(self.rt.device) - before)
            self.graphs_recorded += 1
        self._graphs[key] = rec                                # dicts keep insertion order: the oldest use comes first
        while len(self._graphs) > 1 and (len(self._graphs) > self.MAX_GRAPHS or self.graph_bytes() > self.graph_memory_bytes):
            self._graphs.pop(next(iter(self._graphs)))
        return rec

    def graph_bytes(self) -> int:
        """Device memory that the recorded steps hold (their buffers, activations and workspaces)."""
        return sum(r["bytes"] for r in self._graphs.values())

    # ---- requests ------------------------------------------------------------------
    def add_request(self, req_id: Hashable):
        return self.cache.add_request(req_id)

    def free_request(self, req_id: Hashable) -> None:
        self.cache.free_request(req_id)
        self._poison_pages()

    def _begin_new_requests(self, seqs: Sequence[SeqInfo]) -> None:
        """For a request that runs its first step: its fixed-size state begins at zero, and its entry of
        ``shared_keys`` says how many of its first keys lie in pages that it took over from other requests
        (the request that computed them first is not told: one reader of many)."""
        for s in seqs:
            if s.new_request:
                for st in self.state:
                    if st is not None:
                        st[s.state_slot].zero_()
                shared = self.cache.get(s.req_id).shared_len
                if self._shared_keys_host[s.state_slot] != shared:
                    self._shared_keys_host[s.state_slot] = shared
                    self.shared_keys[s.state_slot:s.state_slot + 1].fill_(shared)

    def _poison_pages(self) -> None:
        """With debug_poison: NaN into every page that was handed out or went back since the last
        call (plain fills on the current stream, outside any recorded graph)."""
        if not self.debug_poison:
            return
        events = self.cache.take_page_events()
        if not events:
            return
        by_group = {}
        for g, page in events:
            by_group.setdefault(g, set()).add(page)
        for g, pages in by_group.items():
            idx = torch.tensor(sorted(pages), dtype=torch.long, device=self.rt.device)
            for i, kv in enumerate(self.kv):
                if kv is not None and self.plan.user_group[i] == g:
                    kv.index_fill_(0, idx, float("nan"))
            self.pages_poisoned += len(pages)

    def _check_bounds(self, seqs: Sequence[SeqInfo], slots: List[np.ndarray], upd_idx: List[np.ndarray],
                      upd_val: List[np.ndarray]) -> None:
        """Host check of what a step sends to the device: every cache slot and every table entry
        lies inside its pool and its table; with debug_poison also that each request holds a page
        for every position its tokens can see."""
        P = self.page_size
        for g, pool in enumerate(self.cache.pools):
            if len(slots[g]) and (int(slots[g].min()) < -1 or int(slots[g].max()) >= pool.num_pages * P):
                raise RuntimeError(f"a cache slot of group {g} lies outside its {pool.num_pages} pages")
            if len(upd_val[g]) and (int(upd_val[g].min()) < -1 or int(upd_val[g].max()) >= pool.num_pages):
                raise RuntimeError(f"a table entry of group {g} names a page outside its {pool.num_pages} pages")
            if len(upd_idx[g]) and (int(upd_idx[g].min()) < 0 or
                                    int(upd_idx[g].max()) >= self.max_requests * self.table_width[g]):
                raise RuntimeError(f"a table update of group {g} lies outside the requests' table rows")
        if not self.debug_poison:
            return
        for s in seqs:
            if s.req_id is None:
                continue
            rc = self.cache.get(s.req_id)
            for g, grp in enumerate(self.cache.groups):
                first_key = 0 if grp.window is None else max(0, s.kv_before - grp.window + 1)
                last_key = s.kv_before + s.q_len - 1
                table = rc.tables[g]
                for i in range(first_key // P, last_key // P + 1):
                    if i >= len(table) or table[i] < 0:
                        raise RuntimeError(f"request {s.req_id!r} holds no page for position {i * P} of group {g}, "
                                           f"which its tokens at {s.kv_before}..{last_key} can see")

    def cache_bytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in self.kv if t is not None)

    # ---- one step ----------------------------------------------------------------------
    def _check_and_reserve(self, entries: Sequence[StepEntry]) -> List[np.ndarray]:
        """Checks the entries, reserves their pages (all or none), and returns the entries'
        tokens as int32 arrays."""
        cache = self.cache
        vocab = self.model.spec.vocab_size
        max_pos = self.model.spec.max_positions
        if not entries:
            raise ValueError("a step needs at least one entry")
        seen = set()
        tokens: List[np.ndarray] = []
        for e in entries:
            if e.req_id in seen:
                raise ValueError(f"request {e.req_id!r} appears twice in one step")
            seen.add(e.req_id)
            if len(e.tokens) == 0:
                raise ValueError(f"request {e.req_id!r} brings no tokens")
            arr = np.asarray(e.tokens)
            if arr.ndim != 1 or arr.dtype.kind not in "iu":
                raise ValueError(f"the tokens of request {e.req_id!r} are not a flat list of integers")
            bad = (arr < 0) | (arr >= vocab)
            if bad.any():
                raise ValueError(f"token id {int(arr[bad][0])} of request {e.req_id!r} is outside the "
                                 f"vocabulary of {vocab}")
            tokens.append(arr.astype(np.int32))
            for w in e.want:
                if not 0 <= int(w) < len(e.tokens):
                    raise ValueError(f"request {e.req_id!r} wants logits at place {w} of {len(e.tokens)} tokens")
            rc = cache.get(e.req_id)
            if rc.num_tokens + len(e.tokens) > max_pos:
                raise ValueError(f"request {e.req_id!r} would pass the model's {max_pos} positions")
        if not cache.can_reserve([(e.req_id, cache.get(e.req_id).num_tokens + len(e.tokens)) for e in entries]):
            raise OutOfPages("the cache has too few free pages for this step")
        for e in entries:
            cache.reserve(e.req_id, cache.get(e.req_id).num_tokens + len(e.tokens))
        return tokens

    def _layout(self, entries: Sequence[StepEntry], tokens: List[np.ndarray]):
        """The batch as flat int32 host arrays: (seqs, token ids, positions, table row of each
        token, wanted rows, and per group: cache slot of each token, changed table entries)."""
        cache = self.cache
        seqs: List[SeqInfo] = []
        positions, tok_seq, rows = [], [], []
        n_groups = len(cache.groups)
        slots: List[list] = [[] for _ in range(n_groups)]
        upd_idx: List[List[int]] = [[] for _ in range(n_groups)]
        upd_val: List[List[int]] = [[] for _ in range(n_groups)]
        q_start = 0
        for e, tok in zip(entries, tokens):
            rc = cache.get(e.req_id)
            n = len(tok)
            seqs.append(SeqInfo(e.req_id, q_start, n, rc.num_tokens, rc.state_slot, rc.new_request))
            positions.append(np.arange(rc.num_tokens, rc.num_tokens + n, dtype=np.int32))
            tok_seq.append(np.full(n, rc.state_slot, dtype=np.int32))   # the request's row in the device tables
            rows.append(np.asarray(e.want, dtype=np.int32).reshape(-1) + q_start)
            for g in range(n_groups):
                slots[g].append(cache.token_slot_array(e.req_id, g, rc.num_tokens, n))
                width = self.table_width[g]
                for i, page in cache.take_dirty(e.req_id, g):
                    if i >= width:
                        raise RuntimeError("a request holds more pages than its table row has entries")
                    upd_idx[g].append(rc.state_slot * width + i)
                    upd_val[g].append(page)
            q_start += n
        cat = np.concatenate
        return (seqs, cat(tokens), cat(positions), cat(tok_seq), cat(rows), [cat(x) for x in slots],
                [np.asarray(u, dtype=np.int32) for u in upd_idx], [np.asarray(u, dtype=np.int32) for u in upd_val])

    def _single_token_layout(self, entries: Sequence[StepEntry]):
        """What _check_and_reserve and _layout do, for entries of one token each, with plain
        integers: a decode step's host time is per request, and an array per request costs
        more than the request's whole bookkeeping."""
        cache = self.cache
        vocab, max_pos, P = self.model.spec.vocab_size, self.model.spec.max_positions, self.page_size
        n_groups = len(cache.groups)
        seen = set()
        rcs, wants = [], []
        for e in entries:
            if e.req_id in seen:
                raise ValueError(f"request {e.req_id!r} appears twice in one step")
            seen.add(e.req_id)
            t = e.tokens[0]
            if not isinstance(t, (int, np.integer)) or not 0 <= t < vocab:
                raise ValueError(f"token id {t} of request {e.req_id!r} is outside the vocabulary of {vocab}")
            rc = cache.get(e.req_id)
            if rc.num_tokens + 1 > max_pos:
                raise ValueError(f"request {e.req_id!r} would pass the model's {max_pos} positions")
            rcs.append(rc)
            if any(len(table) * P <= rc.num_tokens for table in rc.tables):   # its next position has no page yet
                wants.append((e.req_id, rc.num_tokens + 1))
        if wants:
            if not cache.can_reserve(wants):
                raise OutOfPages("the cache has too few free pages for this step")
            for req_id, new_len in wants:
                cache.reserve(req_id, new_len)
        B = len(entries)
        seqs = []
        tok, pos, seq = [0] * B, [0] * B, [0] * B
        slots = [[0] * B for _ in range(n_groups)]
        upd_idx: List[List[int]] = [[] for _ in range(n_groups)]
        upd_val: List[List[int]] = [[] for _ in range(n_groups)]
        for i, (e, rc) in enumerate(zip(entries, rcs)):
            n = rc.num_tokens
            seqs.append(SeqInfo(e.req_id, i, 1, n, rc.state_slot, rc.new_request))
            tok[i], pos[i], seq[i] = int(e.tokens[0]), n, rc.state_slot
            for g in range(n_groups):
                page = rc.tables[g][n // P]
                if page < 0:
                    raise RuntimeError(f"request {e.req_id!r} holds no page for position {n} in group {g}")
                slots[g][i] = page * P + n % P
                if rc.dirty[g]:
                    width = self.table_width[g]
                    for j, pg in cache.take_dirty(e.req_id, g):
                        if j >= width:
                            raise RuntimeError("a request holds more pages than its table row has entries")
                        upd_idx[g].append(rc.state_slot * width + j)
                        upd_val[g].append(pg)
        i32 = np.int32
        return (seqs, np.asarray(tok, dtype=i32), np.asarray(pos, dtype=i32), np.asarray(seq, dtype=i32),
                np.arange(B, dtype=i32), [np.asarray(x, dtype=i32) for x in slots],
                [np.asarray(u, dtype=i32) for u in upd_idx], [np.asarray(u, dtype=i32) for u in upd_val])

    def _to_device(self, parts: List[np.ndarray]) -> List[torch.Tensor]:
        """One copy of all the arrays to the device, through a pinned buffer that is kept and grown;
        returns a device view for each part."""
        total = sum(len(x) for x in parts)
        if self._stage is None or self._stage.numel() < total:
            self._stage = torch.empty(max(total, 4096), dtype=torch.int32).pin_memory()
            self._stage_np = self._stage.numpy()
        else:
            self._stage_event.synchronize()               # the last copy out of the buffer is done
        np.concatenate(parts, out=self._stage_np[:total])
        dev = self._stage[:total].to(self.rt.device, non_blocking=True)
        self._stage_event.record()
        out, off = [], 0
        for x in parts:
            out.append(dev[off:off + len(x)])
            off += len(x)
        return out

    def build_context(self, entries: Sequence[StepEntry]) -> StepContext:
        """Reserves pages for the entries' tokens, lays the batch out flat, and brings the
        device's block tables up to date (one copy to the device, one small kernel per group)."""
        tokens = self._check_and_reserve(entries)
        seqs, token_ids, positions, tok_seq, rows, slots, upd_idx, upd_val = self._layout(entries, tokens)
        self._check_bounds(seqs, slots, upd_idx, upd_val)
        self._poison_pages()                       # (the pages just handed out, before anything is written)
        T, n_groups = len(token_ids), len(self.cache.groups)
        i32 = np.int32
        parts = [token_ids, positions, tok_seq, rows, np.asarray([s.state_slot for s in seqs], dtype=i32)]
        n_fixed = len(parts)
        for g in range(n_groups):
            parts += [slots[g], upd_idx[g], upd_val[g]]
        # what single parts want prepared for the step: their arrays travel in the same copy
        extras = {cls: dict(cls.step_extras(seqs)) for cls in self._step_classes}
        wanted = [(cls, name) for cls, d in extras.items() for name, v in d.items() if isinstance(v, np.ndarray)]
        parts += [extras[cls][name].astype(i32, copy=False) for cls, name in wanted]
        dev = self._to_device(parts)
        d_tok, d_pos, d_seq, d_rows, d_state = dev[:n_fixed]
        d_slots = []
        for g in range(n_groups):
            d_slot, d_idx, d_val = dev[n_fixed + 3 * g:n_fixed + 3 + 3 * g]
            d_slots.append(d_slot)
            if len(d_idx):
                ops.scatter_int(self.tables[g], d_idx, d_val)
        for (cls, name), t in zip(wanted, dev[n_fixed + 3 * n_groups:]):
            extras[cls][name] = t
        return StepContext(rt=self.rt, page_size=self.page_size, num_tokens=T, seqs=seqs, token_ids=d_tok,
                           positions=d_pos, tok_seq=d_seq, block_tables=self.tables,
                           shared_keys=self.shared_keys, slots=d_slots,
                           logit_rows=d_rows, state_slots=d_state, max_position=int(positions.max()),
                           extras=extras)

    def step(self, entries: Sequence[StepEntry], greedy: bool = False):
        """Runs the entries' tokens as one batch; returns float32 logits [wanted, vocab] on the
        device, in the order of the entries and of their ``want``.  With ``greedy`` it returns, instead,
        the index of the largest logit of every wanted row (the lowest on ties, src/engine/executor.py:51-54)
        as a list of integers: a recorded step picks them inside its graph, and no logits travel."""
        logits = None
        if self.use_graphs and all(len(e.tokens) == 1 and list(e.want) == [0] for e in entries) and entries:
            logits = self._decode_step_with_graph(entries, greedy)
        elif self.use_graphs and self._portion_graphs and len(entries) == 1 and len(entries[0].want) <= 1 and \
                len(entries[0].tokens) >= self.PORTION_GRAPH_MIN and len(entries[0].tokens) % self.PORTION_GRAPH_STEP == 0:
            logits = self._portion_step_with_graph(entries[0], greedy)
        elif self.use_graphs and self._mixed_graphs and self._is_mixed_step(entries):
            logits = self._mixed_step_with_graph(entries, greedy)
        if logits is None:                         # (also a shape that is not recorded yet)
            ctx = self.build_context(entries)
            self._begin_new_requests(ctx.seqs)
            logits = self.model.forward(ctx, self.bindings)
            if greedy:
                logits = ops.argmax(logits).tolist() if logits.shape[0] else []
        for e in entries:
            self.cache.commit(e.req_id, e.tokens)
        self._poison_pages()                       # (pages that a window has passed went back)
        self.steps_run += 1
        return logits

    # ---- decoding through a recorded graph ------------------------------------------------
    def _recorded_argmax(self, logits: torch.Tensor) -> Optional[torch.Tensor]:
        """Inside a recording: the largest logit's index of every row, into a buffer that stays (through the
        entry point that allocates nothing, where the rows fit its buffer)."""
        if logits.shape[0] == 0:
            return None
        tokens = torch.empty(logits.shape[0], dtype=torch.int32, device=logits.device)
        if ops.argmax_static_takes(*logits.shape):
            return ops.argmax_static(logits, tokens)
        return ops.argmax(logits, out=tokens)

    def _decode_step_with_graph(self, entries: Sequence[StepEntry], greedy: bool = False):
        seqs, token_ids, positions, tok_seq, rows, slots, upd_idx, upd_val = self._single_token_layout(entries)
        self._check_bounds(seqs, slots, upd_idx, upd_val)
        self._poison_pages()                       # (the pages just handed out, before anything is written)
        self._begin_new_requests(seqs)
        n_live, n_groups = len(seqs), len(self.cache.groups)
        i32 = np.int32
        # Graphs are recorded for 1 to 8 rows, for multiples of 8 and, beyond 64, of 32: a batch in between is filled up
        # with rows that stand at position 0 of the tables' spare row, write nowhere (cache slot
        # -1) and whose logits are dropped, so that a batch that shrinks request by request does not
        # record a graph for every size it passes.
        B = self.graph_rows(n_live)
        if B > n_live:
            fill = B - n_live
            token_ids = np.concatenate([token_ids, np.zeros(fill, dtype=i32)])
            positions = np.concatenate([positions, np.zeros(fill, dtype=i32)])
            tok_seq = np.concatenate([tok_seq, np.full(fill, self.spare_row, dtype=i32)])
            slots = [np.concatenate([x, np.full(fill, -1, dtype=i32)]) for x in slots]
        cap = 2 * B                                    # table updates a decode step can bring per group
        max_position = int(positions.max())
        part_keys = tuple(cls.graph_key(max_position) if hasattr(cls, "graph_key") else None
                          for cls in self._step_classes)
        if any(len(u) > cap for u in upd_idx):
            # more table changes than the recorded step takes (the first decode step after a
            # preemption, say): bring the tables up to date apart, then go on with none
            for g in range(n_groups):
                if len(upd_idx[g]):
                    ops.scatter_int(self.tables[g], torch.from_numpy(upd_idx[g]).to(self.rt.device),
                                    torch.from_numpy(upd_val[g]).to(self.rt.device))
                upd_idx[g] = upd_val[g] = np.zeros(0, dtype=i32)
        rec = self._graph_for((B, part_keys), "decode", lambda: self._record_decode_graph(B, part_keys, cap))
        iota, none, zero = rec["iota"], rec["none"], rec["zero"]       # 0 .. B - 1; cap times -1; cap zeros
        # (a row's table row is its request's state slot: tok_seq serves as both)
        parts = [token_ids, positions, tok_seq, iota, tok_seq]
        for g in range(n_groups):
            pad = cap - len(upd_idx[g])
            parts += [slots[g], upd_idx[g], none[:pad], upd_val[g], zero[:pad]]
        rec["event"].synchronize()                     # the last copy out of the host buffer is done
        np.concatenate(parts, out=rec["host_np"])
        rec["meta"].copy_(rec["host"], non_blocking=True)
        rec["event"].record()
        rec["graph"].replay()
        self.graph_steps += 1
        self.graph_steps_of["decode"] += 1
        if greedy:
            return rec["tokens"].tolist()[:n_live]      # (one small copy to the host; waits for the step)
        return rec["logits"][:n_live].clone()          # the graph's own output is overwritten by the next replay

    # ---- single new tokens beside one prompt portion through a recorded graph -----------------
    def _is_mixed_step(self, entries: Sequence[StepEntry]) -> bool:
        """Single tokens that want their logits, and exactly one portion of 2 to MIXED_GRAPH_MAX_TOKENS
        tokens that wants its last row's logits or none."""
        portion = None
        for e in entries:
            n = len(e.tokens)
            if n == 1:
                if list(e.want) != [0]:
                    return False
            elif portion is not None or n < 2 or n > self.MIXED_GRAPH_MAX_TOKENS or list(e.want) not in ([], [n - 1]) \
                    or -(-n // self.MIXED_GRAPH_STEP) * self.MIXED_GRAPH_STEP > self._spare_positions:
                return False                              # (the rows that fill up, and the stand-in batch, stand at the
            else:                                         # positions 0 .. T - 1 of the spare table row)
                portion = e
        return portion is not None

    def _mixed_step_with_graph(self, entries: Sequence[StepEntry], greedy: bool = False):
        # the single tokens first, the portion last; the logits go back into the entries' order
        order = sorted(range(len(entries)), key=lambda i: len(entries[i].tokens) > 1)
        ordered = [entries[i] for i in order]
        n_dec, n_groups, i32 = len(ordered) - 1, len(self.cache.groups), np.int32
        T1 = len(ordered[-1].tokens)
        B = self.graph_rows(n_dec)
        T = -(-T1 // self.MIXED_GRAPH_STEP) * self.MIXED_GRAPH_STEP
        cap = 2 * B + 2 * (T // self.page_size + 2)
        # which recorded step this is, from the requests' lengths alone (nothing is reserved yet: a shape
        # that is not recorded runs as it comes)
        max_dec_position = max([self.cache.get(e.req_id).num_tokens for e in ordered[:-1]], default=0)
        portion_keys = self.cache.get(ordered[-1].req_id).num_tokens + T1
        part_keys = tuple(cls.mixed_graph_key(max_dec_position, portion_keys) for cls in self._step_classes)
        rec = self._graph_for(("mixed", B, T, part_keys), "mixed", lambda: self._record_mixed_graph(B, T, part_keys, cap))
        if rec is None:
            return None
        tokens = self._check_and_reserve(ordered)
        seqs, token_ids, positions, tok_seq, rows, slots, upd_idx, upd_val = self._layout(ordered, tokens)
        self._check_bounds(seqs, slots, upd_idx, upd_val)
        self._poison_pages()
        self._begin_new_requests(seqs)
        fill, pad = B - n_dec, T - T1
        spare = self.spare_row

        def padded(x, fill_value, pad_values):
            return np.concatenate([x[:n_dec], np.full(fill, fill_value, dtype=i32), pad_values, x[n_dec:]])

        zeros_pad = np.zeros(pad, dtype=i32)
        token_ids = padded(token_ids, 0, zeros_pad)
        positions_all = padded(positions, 0, np.arange(pad, dtype=i32))
        tok_seq = padded(tok_seq, spare, np.full(pad, spare, dtype=i32))
        slots = [padded(x, -1, np.full(pad, -1, dtype=i32)) for x in slots]
        if any(len(u) > cap for u in upd_idx):
            for g in range(n_groups):
                if len(upd_idx[g]):
                    ops.scatter_int(self.tables[g], torch.from_numpy(upd_idx[g]).to(self.rt.device),
                                    torch.from_numpy(upd_val[g]).to(self.rt.device))
                upd_idx[g] = upd_val[g] = np.zeros(0, dtype=i32)
        none, zero = rec["none"], rec["zero"]
        parts = [token_ids, positions_all, tok_seq]
        for g in range(n_groups):
            pad_u = cap - len(upd_idx[g])
            parts += [slots[g], upd_idx[g], none[:pad_u], upd_val[g], zero[:pad_u]]
        for cls in self._step_classes:
            parts.append(np.asarray(cls.mixed_graph_dynamic(B, pad, T), dtype=i32))
        rec["event"].synchronize()
        np.concatenate(parts, out=rec["host_np"])
        rec["meta"].copy_(rec["host"], non_blocking=True)
        rec["event"].record()
        rec["graph"].replay()
        self.graph_steps += 1
        self.graph_steps_of["mixed"] += 1
        # rows of the recorded logits: the B rows of the single tokens, then the portion's last row
        picked = []
        for i in range(len(entries)):
            at = order.index(i)
            if at < n_dec:
                picked.append(at)
            elif entries[i].want:
                picked.append(B)
        if greedy:
            toks = rec["tokens"].tolist()
            return [toks[i] for i in picked]
        logits = rec["logits"]
        if picked == list(range(n_dec)) + [B]:            # the usual order: no index has to travel
            return torch.cat([logits[:n_dec], logits[B:B + 1]]) if n_dec < B else logits[:B + 1].clone()
        if picked == list(range(n_dec)):
            return logits[:n_dec].clone()
        return logits[torch.tensor(picked, dtype=torch.long).to(self.rt.device)]

    def _record_mixed_graph(self, B: int, T: int, part_keys: tuple, cap: int):
        """Static buffers for a step of B single new tokens beside one prompt portion filled up to T
        tokens, one run outside the graph, then the recording.  The stand-in batch: every single token
        at position 0 of the tables' spare row, the portion at its positions 0 .. T - 1, writing nowhere."""
        dev, n_groups = self.rt.device, len(self.cache.groups)
        dyn_sizes = [int(cls.mixed_graph_dynamic_size) for cls in self._step_classes]
        n = 3 * (B + T) + n_groups * (B + T + 2 * cap) + sum(dyn_sizes)
        host = torch.zeros(n, dtype=torch.int32).pin_memory()
        meta = torch.zeros(n, dtype=torch.int32, device=dev)
        stand_in = [0] * (B + T) + [0] * B + list(range(T)) + [self.spare_row] * (B + T)
        for g in range(n_groups):
            stand_in += [-1] * (B + T) + [-1] * cap + [0] * cap
        for cls in self._step_classes:
            stand_in += [int(v) for v in cls.mixed_graph_dynamic(B, 0, T)]
        meta.copy_(torch.tensor(stand_in, dtype=torch.int32))
        off = 0

        def take(k):
            nonlocal off
            t = meta[off:off + k]
            off += k
            return t

        d_tok, d_pos, d_seq = take(B + T), take(B + T), take(B + T)
        d_slots, d_upd = [], []
        for g in range(n_groups):
            d_slots.append(take(B + T))
            d_upd.append((take(cap), take(cap)))
        d_dyn = [take(k) for k in dyn_sizes]
        d_rows = torch.tensor(list(range(B)) + [B + T - 1], dtype=torch.int32, device=dev)
        d_state = torch.full((B + 1,), self.spare_row, dtype=torch.int32, device=dev)
        seqs = [SeqInfo(None, i, 1, 0, self.spare_row, False) for i in range(B)] + \
            [SeqInfo(None, B, T, 0, self.spare_row, False)]
        ctx = StepContext(rt=self.rt, page_size=self.page_size, num_tokens=B + T, seqs=seqs, token_ids=d_tok,
                          positions=d_pos, tok_seq=d_seq, block_tables=self.tables,
                          shared_keys=self.shared_keys, slots=d_slots,
                          logit_rows=d_rows, state_slots=d_state, max_position=0,
                          extras={cls: dict(cls.mixed_graph_extras(B, T, k, dev, dyn))
                                  for cls, k, dyn in zip(self._step_classes, part_keys, d_dyn)})

        def run():
            for g in range(n_groups):
                ops.scatter_int(self.tables[g], d_upd[g][0], d_upd[g][1])
            logits = self.model.forward(ctx, self.bindings)
            return logits, self._recorded_argmax(logits)

        torch.cuda.synchronize()
        stream = torch.cuda.Stream()
        stream.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(stream):
            run()
        stream.synchronize()
        ctx.memo.clear()                          # (what the parts made for the first run is made again inside the graph)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            logits, tokens = run()
        torch.cuda.synchronize()
        event = torch.cuda.Event()
        event.record()
        return {"graph": graph, "ctx": ctx, "host": host, "host_np": host.numpy(), "meta": meta, "logits": logits, "tokens": tokens,
                "event": event, "none": np.full(cap, -1, dtype=np.int32), "zero": np.zeros(cap, dtype=np.int32)}

    # ---- one prompt portion through a recorded graph ----------------------------------------
    def _portion_step_with_graph(self, entry: StepEntry, greedy: bool = False):
        T, n_want, n_groups = len(entry.tokens), len(entry.want), len(self.cache.groups)
        cap = 2 * (T // self.page_size + 2)
        i32 = np.int32
        keys = self.cache.get(entry.req_id).num_tokens + T
        part_keys = tuple(cls.portion_graph_key(T, keys) if hasattr(cls, "portion_graph_key") else None
                          for cls in self._step_classes)
        rec = self._graph_for(("portion", T, n_want, part_keys), "portion",
                              lambda: self._record_portion_graph(T, n_want, cap, part_keys))
        if rec is None:
            return None
        tokens = self._check_and_reserve([entry])
        seqs, token_ids, positions, tok_seq, rows, slots, upd_idx, upd_val = self._layout([entry], tokens)
        self._check_bounds(seqs, slots, upd_idx, upd_val)
        self._poison_pages()
        self._begin_new_requests(seqs)
        if any(len(u) > cap for u in upd_idx):
            for g in range(n_groups):
                if len(upd_idx[g]):
                    ops.scatter_int(self.tables[g], torch.from_numpy(upd_idx[g]).to(self.rt.device),
                                    torch.from_numpy(upd_val[g]).to(self.rt.device))
                upd_idx[g] = upd_val[g] = np.zeros(0, dtype=i32)
        none, zero = rec["none"], rec["zero"]
        parts = [token_ids, positions, tok_seq, rows, np.asarray([seqs[0].state_slot], dtype=i32)]
        for g in range(n_groups):
            pad = cap - len(upd_idx[g])
            parts += [slots[g], upd_idx[g], none[:pad], upd_val[g], zero[:pad]]
        rec["event"].synchronize()
        np.concatenate(parts, out=rec["host_np"])
        rec["meta"].copy_(rec["host"], non_blocking=True)
        rec["event"].record()
        rec["graph"].replay()
        self.graph_steps += 1
        self.graph_steps_of["portion"] += 1
        if greedy:
            return rec["tokens"].tolist() if rec["tokens"] is not None else []
        return rec["logits"].clone()

    def _record_portion_graph(self, T: int, n_want: int, cap: int, part_keys: tuple):
        """Static buffers for a step that is one prompt portion of T tokens with n_want (0 or 1) rows
        of logits, at a place that gives the parts' ``part_keys``, one run outside the graph, then the
        recording.  The stand-in batch stands at
        positions 0 .. T - 1 of the tables' spare row (every entry page 0) and writes nowhere."""
        dev, n_groups = self.rt.device, len(self.cache.groups)
        n = 3 * T + n_want + 1 + n_groups * (T + 2 * cap)
        host = torch.zeros(n, dtype=torch.int32).pin_memory()
        meta = torch.zeros(n, dtype=torch.int32, device=dev)
        stand_in = [0] * T + list(range(T)) + [self.spare_row] * T + [T - 1] * n_want + [self.spare_row]
        for g in range(n_groups):
            stand_in += [-1] * T + [-1] * cap + [0] * cap
        meta.copy_(torch.tensor(stand_in, dtype=torch.int32))
        off = 0

        def take(k):
            nonlocal off
            t = meta[off:off + k]
            off += k
            return t

        d_tok, d_pos, d_seq, d_rows, d_state = take(T), take(T), take(T), take(n_want), take(1)
        d_slots, d_upd = [], []
        for g in range(n_groups):
            d_slots.append(take(T))
            d_upd.append((take(cap), take(cap)))
        seqs = [SeqInfo(None, 0, T, 0, self.spare_row, False)]
        ctx = StepContext(rt=self.rt, page_size=self.page_size, num_tokens=T, seqs=seqs, token_ids=d_tok,
                          positions=d_pos, tok_seq=d_seq, block_tables=self.tables,
                          shared_keys=self.shared_keys, slots=d_slots,
                          logit_rows=d_rows, state_slots=d_state, max_position=0,
                          extras={cls: dict(cls.portion_graph_extras(T, dev) if k is None
                                            else cls.portion_graph_extras(T, dev, k))
                                  for cls, k in zip(self._step_classes, part_keys)})

        def run():
            for g in range(n_groups):
                ops.scatter_int(self.tables[g], d_upd[g][0], d_upd[g][1])
            logits = self.model.forward(ctx, self.bindings)
            return logits, self._recorded_argmax(logits)

        torch.cuda.synchronize()
        stream = torch.cuda.Stream()
        stream.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(stream):
            run()                                 # (what the parts keep for the step, ctx.memo, is made here)
        stream.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            logits, tokens = run()
        torch.cuda.synchronize()
        event = torch.cuda.Event()
        event.record()
        return {"graph": graph, "ctx": ctx, "host": host, "host_np": host.numpy(), "meta": meta, "logits": logits, "tokens": tokens,
                "event": event, "none": np.full(cap, -1, dtype=np.int32), "zero": np.zeros(cap, dtype=np.int32)}

    def _record_decode_graph(self, B: int, part_keys: tuple, cap: int):
        """Static buffers for a decode step of B requests whose positions give the parts'
        ``part_keys``, one run outside the graph (so that nothing is set up for the first time
        while recording), then the recording."""
        dev, n_groups = self.rt.device, len(self.cache.groups)
        n = 5 * B + n_groups * (B + 2 * cap)
        host = torch.zeros(n, dtype=torch.int32).pin_memory()
        meta = torch.zeros(n, dtype=torch.int32, device=dev)
        # a harmless stand-in batch for the runs that only record: every token at position 0 of
        # the tables' spare row, writing nowhere (cache slot -1), no table updates
        stand_in = [0] * (2 * B) + [self.spare_row] * B + list(range(B)) + [self.spare_row] * B
        for g in range(n_groups):
            stand_in += [-1] * B + [-1] * cap + [0] * cap
        meta.copy_(torch.tensor(stand_in, dtype=torch.int32))
        off = 0

        def take(k):
            nonlocal off
            t = meta[off:off + k]
            off += k
            return t

        d_tok, d_pos, d_seq, d_rows, d_state = (take(B) for _ in range(5))
        d_slots, d_upd = [], []
        for g in range(n_groups):
            d_slots.append(take(B))
            d_upd.append((take(cap), take(cap)))
        seqs = [SeqInfo(None, i, 1, 0, 0, False) for i in range(B)]
        ctx = StepContext(rt=self.rt, page_size=self.page_size, num_tokens=B, seqs=seqs, token_ids=d_tok,
                          positions=d_pos, tok_seq=d_seq, block_tables=self.tables,
                          shared_keys=self.shared_keys, slots=d_slots,
                          logit_rows=d_rows, state_slots=d_state, max_position=0,
                          extras={cls: dict(cls.graph_extras(B, k, dev)) if hasattr(cls, "graph_extras") else {}
                                  for cls, k in zip(self._step_classes, part_keys)})

        def run():
            for g in range(n_groups):
                ops.scatter_int(self.tables[g], d_upd[g][0], d_upd[g][1])
            logits = self.model.forward(ctx, self.bindings)
            return logits, self._recorded_argmax(logits)

        torch.cuda.synchronize()
        stream = torch.cuda.Stream()
        stream.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(stream):
            run()
        stream.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            logits, tokens = run()
        torch.cuda.synchronize()
        event = torch.cuda.Event()
        event.record()
        # (the context is kept with the graph: what the parts made for the recorded step, their
        # graph_extras, is read by every replay)
        return {"graph": graph, "ctx": ctx, "host": host, "host_np": host.numpy(), "meta": meta, "logits": logits, "tokens": tokens,
                "event": event, "iota": np.arange(B, dtype=np.int32), "none": np.full(cap, -1, dtype=np.int32),
                "zero": np.zeros(cap, dtype=np.int32)}
