"""From a model's schedule to cache groups: which parts of which schedule entries keep keys
and values, with which window, and which keep per-request state of fixed size."""
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
    """A *cache user* is one part of a block that keeps keys and values, or state of fixed size, or reads
    another user's cache: a block with one mixer has one user per schedule entry, a block with two
    mixers side by side two, a block without a mixer none.  Users are numbered in the order of the
    schedule, and inside an entry in the order in which the block's forward gets their bindings."""
    groups: List[GroupSpec]                  # distinct needs, in order of first use
    entry_users: List[List[int]]             # per schedule entry: its cache users
    user_group: List[Optional[int]]          # per user: its group (also for users that read another's cache)
    user_kv: List[Optional[KVNeed]]          # per user: storage it owns, None if it owns none
    user_source: List[Optional[int]]         # per user: the user whose storage it uses (itself if it owns one)
    user_state: List[Optional[StateNeed]]    # per user: fixed-size state

    def bytes_per_token(self, itemsize: int) -> int:
        return sum(2 * kv.num_kv_heads * kv.head_dim * itemsize for kv in self.user_kv if kv is not None)


Need = Tuple[Optional[KVNeed], Optional[StateNeed]]


def plan_cache(entry_needs: Sequence[tuple]) -> CachePlan:
    """entry_needs[i] describes schedule entry i: (needs, cache_from), needs being the list of
    (kv need, state need) of the entry's block, one per cache user; or, for a block with one user,
    (kv need, state need, cache_from).  An entry that reads the cache of an earlier entry pairs its
    users with that entry's, one by one."""
    groups: List[GroupSpec] = []
    entry_users: List[List[int]] = []
    user_group: List[Optional[int]] = []
    user_kv: List[Optional[KVNeed]] = []
    user_source: List[Optional[int]] = []
    user_state: List[Optional[StateNeed]] = []
    for i, item in enumerate(entry_needs):
        needs, cache_from = ([(item[0], item[1])], item[2]) if len(item) == 3 else (list(item[0]), item[1])
        if cache_from is not None and len(entry_users[cache_from]) != len(needs):
            raise ValueError(f"schedule entry {i} has {len(needs)} cache users, entry {cache_from}, whose cache "
                             f"it reads, has {len(entry_users[cache_from])}")
        users = []
        for j, (kv, state) in enumerate(needs):
            u = len(user_kv)
            users.append(u)
            user_state.append(state)
            if cache_from is not None:
                src = entry_users[cache_from][j]
                src_kv = user_kv[src]
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
                user_kv.append(None)
                user_source.append(src if src_kv is not None else None)
                user_group.append(user_group[src])
                continue
            if kv is None:
                user_kv.append(None)
                user_source.append(None)
                user_group.append(None)
                continue
            spec = GroupSpec(window=kv.window)
            if spec not in groups:
                groups.append(spec)
            user_kv.append(kv)
            user_source.append(u)
            user_group.append(groups.index(spec))
        entry_users.append(users)
    return CachePlan(groups, entry_users, user_group, user_kv, user_source, user_state)
