"""From a model's schedule to cache groups: which schedule entries keep keys and
values, with which window, and which keep per-request state of fixed size."""
from __future__ import annotations

from dataclasses import dataclass
from typing import List, Optional, Sequence, Tuple

from .manager import GroupSpec


@dataclass(frozen=True)
class KVNeed:
    """Keys and values of every position (window None) or of the last ``window``."""
    num_kv_heads: int
    head_dim: int
    window: Optional[int] = None


@dataclass(frozen=True)
class StateNeed:
    """A tensor of this shape per live request, cleared when the request starts."""
    shape: Tuple[int, ...]
    dtype: str = "float32"


@dataclass
class CachePlan:
    groups: List[GroupSpec]                  # distinct needs, in order of first use
    entry_group: List[Optional[int]]         # per schedule entry: its group (also for entries that read another's cache)
    entry_kv: List[Optional[KVNeed]]         # per schedule entry: storage it owns, None if it owns none
    entry_source: List[Optional[int]]        # per schedule entry: the entry whose storage it uses (itself if it owns one)
    entry_state: List[Optional[StateNeed]]   # per schedule entry: fixed-size state

    def bytes_per_token(self, itemsize: int) -> int:
        return sum(2 * kv.num_kv_heads * kv.head_dim * itemsize for kv in self.entry_kv if kv is not None)


def plan_cache(entry_needs: Sequence[Tuple[Optional[KVNeed], Optional[StateNeed], Optional[int]]]) -> CachePlan:
    """entry_needs[i] = (kv need, state need, cache_from) of schedule entry i."""
    groups: List[GroupSpec] = []
    entry_group: List[Optional[int]] = []
    entry_kv: List[Optional[KVNeed]] = []
    entry_source: List[Optional[int]] = []
    entry_state: List[Optional[StateNeed]] = []
    for i, (kv, state, cache_from) in enumerate(entry_needs):
        entry_state.append(state)
        if cache_from is not None:
            src_kv = entry_kv[cache_from]
            if kv is not None and src_kv is not None and \
                    (kv.num_kv_heads, kv.head_dim) != (src_kv.num_kv_heads, src_kv.head_dim):
                raise ValueError(f"schedule entry {i} cannot read the cache of entry {cache_from}: "
                                 f"their key/value shapes differ")
            if kv is not None and src_kv is not None and src_kv.window is not None and \
                    (kv.window is None or kv.window > src_kv.window):
                # the source's group gives pages back once its own window has passed them: a reader
                # that looks further back would read pages that are no longer the request's
                raise ValueError(f"schedule entry {i} (window {kv.window}) cannot read the cache of entry "
                                 f"{cache_from}, which keeps only the last {src_kv.window} keys")
            entry_kv.append(None)
            entry_source.append(cache_from if src_kv is not None else None)
            entry_group.append(entry_group[cache_from])
            continue
        if kv is None:
            entry_kv.append(None)
            entry_source.append(None)
            entry_group.append(None)
            continue
        spec = GroupSpec(window=kv.window)
        if spec not in groups:
            groups.append(spec)
        entry_kv.append(kv)
        entry_source.append(i)
        entry_group.append(groups.index(spec))
    return CachePlan(groups, entry_group, entry_kv, entry_source, entry_state)
