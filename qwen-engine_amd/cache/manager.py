"""Cache manager: pages of keys and values, a block table for each request, and
slots for per-request state of fixed size.  Pure host code, no tensors.

Layers with the same need form a *group* (all earlier keys, or a window of the
most recent ones).  A group has its own page pool; a page id addresses the same
page in the storage of every layer of the group.  A request holds, per group, a
table from page index (position // page_size) to page id, with -1 where it holds
no page (never allocated, or given back because a window has passed it).

What the reference does and this keeps: a LIFO free list that hands out page 0
first (src/engine/kvcache.py:67,149-154,166), reference counts with retain and
release (kvcache.py:127-147), and a hash chain over full pages for sharing a
common prefix between requests (kvcache.py:81-125).  What differs: pages go back
when a request ends (the reference waits for the whole queue, llm_engine.py:147-152);
a page is registered for sharing only once all its tokens are computed, and the map
from page to hash is kept, so that a freed page leaves the registry
(kvcache.py:163-165 pops a map that nothing fills); a reservation is all or nothing.

With ``keep_freed_prefixes`` the registered pages of a request that ends are not freed at once:
they stay registered, held by nobody, until a later request with the same beginning takes them
over or a reservation needs their memory (then the one kept longest goes first, and of one
request's pages the last before the first, so that no kept page outlives the pages before it).
"""
from __future__ import annotations

import hashlib
import random
from collections import OrderedDict
from dataclasses import dataclass, field
from typing import Dict, Hashable, List, Optional, Sequence, Tuple

import numpy as np


class CacheError(RuntimeError):
    """A request for pages or slots that cannot be met, or a misuse of the manager."""


class OutOfPages(CacheError):
    pass


@dataclass(frozen=True)
class GroupSpec:
    """The need of a group of layers: ``window`` None keeps every key, an int
    keeps the ``window`` most recent positions (the current one included)."""
    window: Optional[int] = None


class PagePool:
    """Pages of one group: LIFO free list and reference counts.

    scatter: the pages are first handed out in a fixed pseudo-random order instead of 0, 1, 2, ...:
    aligned runs of SCATTER_RUN neighbouring pages stay together and in order, the runs are shuffled.
    Handed out in order, the pages that a decode step reads together (the same place of every
    request and of every split of its keys) lie at regular distances in memory, and how well the
    memory serves them then depends on those distances: eight requests of 4096 tokens decoded in
    1.75 to 1.94 ms a step depending on how many pages each prompt had taken (248 or 250), against
    1.76 to 1.78 ms whatever the prompts' lengths with the pages scattered (runs of 32 pages were the
    best of 1, 8, 16, 32 and 64, by a percent).  A pool that has served requests for a while is
    scattered anyway; this makes a fresh one behave the same."""

    SCATTER_RUN = 32

    def __init__(self, num_pages: int, scatter: bool = False):
        if num_pages <= 0:
            raise CacheError("a page pool needs at least one page")
        self.num_pages = num_pages
        self.free: List[int] = list(range(num_pages - 1, -1, -1))  # pop() hands out 0 first
        if scatter:
            groups = [list(range(a, min(a + self.SCATTER_RUN, num_pages))) for a in range(0, num_pages, self.SCATTER_RUN)]
            random.Random(0x5ca77e6).shuffle(groups)
            self.free = [p for grp in groups for p in grp][::-1]
        self.refcount: List[int] = [0] * num_pages

    @property
    def num_free(self) -> int:
        return len(self.free)

    def allocate(self) -> int:
        if not self.free:
            raise OutOfPages("no free page")
        page = self.free.pop()
        if self.refcount[page] != 0:
            raise CacheError(f"free page {page} has reference count {self.refcount[page]}")
        self.refcount[page] = 1
        return page

    def retain(self, page: int) -> None:
        self._check_id(page)
        if self.refcount[page] <= 0:
            raise CacheError(f"cannot retain page {page}: it is free")
        self.refcount[page] += 1

    def release(self, page: int, to_free_list: bool = True) -> bool:
        """Drop one reference; True if nobody holds the page any more (it then goes to the free
        list, unless the caller keeps it aside)."""
        self._check_id(page)
        if self.refcount[page] <= 0:
            raise CacheError(f"cannot release page {page}: it is free already")
        self.refcount[page] -= 1
        if self.refcount[page] == 0:
            if to_free_list:
                self.free.append(page)
            return True
        return False

    def revive(self, page: int) -> None:
        """A page that was kept aside with no holder gets its first holder again."""
        self._check_id(page)
        if self.refcount[page] != 0:
            raise CacheError(f"page {page} is held: it cannot be revived")
        self.refcount[page] = 1

    def give_back(self, page: int) -> None:
        """A page that was kept aside with no holder goes to the free list."""
        self._check_id(page)
        if self.refcount[page] != 0:
            raise CacheError(f"page {page} is held: it cannot be given back")
        self.free.append(page)

    def _check_id(self, page: int) -> None:
        if not 0 <= page < self.num_pages:
            raise CacheError(f"page id {page} is outside 0..{self.num_pages - 1}")


class StateSlots:
    """Slots for per-request state of fixed size: one index per live request."""

    def __init__(self, num_slots: int):
        if num_slots <= 0:
            raise CacheError("at least one state slot is needed")
        self.num_slots = num_slots
        self.free: List[int] = list(range(num_slots - 1, -1, -1))
        self.owner: List[Optional[Hashable]] = [None] * num_slots

    @property
    def num_free(self) -> int:
        return len(self.free)

    def take(self, owner: Hashable) -> int:
        if not self.free:
            raise CacheError("no free state slot")
        slot = self.free.pop()
        self.owner[slot] = owner
        return slot

    def give_back(self, slot: int) -> None:
        if not 0 <= slot < self.num_slots or self.owner[slot] is None:
            raise CacheError(f"state slot {slot} is not held")
        self.owner[slot] = None
        self.free.append(slot)


def chain_hash(parent: int, tokens: Sequence[int]) -> int:
    """64-bit hash of a page's tokens chained to the hash of the page before it
    (the construction of src/engine/kvcache.py:81-86)."""
    h = hashlib.blake2b(digest_size=8)
    h.update(int(parent).to_bytes(8, "little", signed=False))
    for tok in tokens:
        h.update(int(tok).to_bytes(8, "little", signed=True))
    return int.from_bytes(h.digest(), "little", signed=False)


@dataclass
class RequestCache:
    """What one live request holds."""
    req_id: Hashable
    state_slot: int
    tables: List[List[int]]            # per group: page index -> page id or -1
    num_tokens: int = 0                # positions whose keys are in the cache
    tokens: List[int] = field(default_factory=list)   # their token ids (for page hashes)
    hashes: List[int] = field(default_factory=list)   # chain hashes of the full pages so far
    shared_len: int = 0                # tokens taken over from other requests at admission
    new_request: bool = True           # no step has run yet: fixed-size state must be cleared
    dirty: List[List[int]] = field(default_factory=list)   # per group: table indices changed since taken
    released: List[int] = field(default_factory=list)      # per group: table entries below this were given back


@dataclass
class _SharedEntry:
    pages: Tuple[int, ...]   # one page id per group
    tokens: Tuple[int, ...]


class CacheManager:
    def __init__(self, groups: Sequence[GroupSpec], num_pages, page_size: int, max_requests: int,
                 prefix_sharing: bool = False, keep_freed_prefixes: bool = False, scatter_pages: bool = False):
        if page_size <= 0:
            raise CacheError("page_size must be positive")
        self.groups = list(groups)
        if isinstance(num_pages, int):
            num_pages = [num_pages] * len(self.groups)
        if len(num_pages) != len(self.groups):
            raise CacheError("one page count per group is needed")
        for g in self.groups:
            if g.window is not None and g.window <= 0:
                raise CacheError("a window must be positive")
        self.page_size = page_size
        self.pools = [PagePool(n, scatter=scatter_pages) for n in num_pages]
        self.slots = StateSlots(max_requests)
        self.requests: Dict[Hashable, RequestCache] = {}
        # a prefix can only be shared when every group keeps all keys
        self.prefix_sharing = bool(prefix_sharing) and bool(self.groups) and \
            all(g.window is None for g in self.groups)
        self._shared: Dict[int, _SharedEntry] = {}
        self._page_hash: Dict[int, int] = {}   # page id of group 0 -> hash it is registered under
        self.keep_freed = bool(keep_freed_prefixes) and self.prefix_sharing
        # registered entries that nobody holds, by hash; the first is the next to go
        self._kept: "OrderedDict[int, _SharedEntry]" = OrderedDict()
        self.stats = {"pages_allocated": 0, "pages_freed": 0, "shared_page_hits": 0, "kept_page_hits": 0,
                      "kept_pages_evicted": 0}
        # with track_pages, every page that is handed out or goes back to a free list is noted as
        # (group, page), for an owner of the storage that wants to overwrite such pages
        self.track_pages = False
        self._page_events: List[Tuple[int, int]] = []

    # ---- requests -------------------------------------------------------------
    def add_request(self, req_id: Hashable) -> RequestCache:
        if req_id in self.requests:
            raise CacheError(f"request {req_id!r} is live already")
        slot = self.slots.take(req_id)
        rc = RequestCache(req_id=req_id, state_slot=slot, tables=[[] for _ in self.groups],
                          dirty=[[] for _ in self.groups], released=[0] * len(self.groups))
        self.requests[req_id] = rc
        return rc

    def get(self, req_id: Hashable) -> RequestCache:
        try:
            return self.requests[req_id]
        except KeyError:
            raise CacheError(f"request {req_id!r} is not live") from None

    def free_request(self, req_id: Hashable) -> None:
        rc = self.get(req_id)
        kept: List[int] = []
        if self.keep_freed:
            # registered pages go index by index, the pages of all groups together: an entry that
            # nobody holds any more is kept instead of freed
            for i, page0 in enumerate(rc.tables[0]):
                h = self._page_hash.get(page0) if page0 >= 0 else None
                entry = self._shared.get(h) if h is not None else None
                if entry is None or any(i >= len(t) or t[i] != entry.pages[g] for g, t in enumerate(rc.tables)):
                    continue
                unheld = [self.pools[g].release(p, to_free_list=False) for g, p in enumerate(entry.pages)]
                if all(unheld):
                    kept.append(h)
                elif any(unheld):
                    raise CacheError("the pages of a shared entry have different counts")
                for t in rc.tables:
                    t[i] = -1
            for h in reversed(kept):               # the request's last page first: it is the first to go
                self._kept[h] = self._shared[h]
        for g, table in enumerate(rc.tables):
            for page in table:
                if page >= 0:
                    self._release(g, page)
            table.clear()
        self.slots.give_back(rc.state_slot)
        del self.requests[req_id]

    # ---- pages ------------------------------------------------------------------
    def _first_live_page(self, g: int, next_pos: int) -> int:
        """Index of the first page that a query at position >= next_pos can still see."""
        w = self.groups[g].window
        if w is None:
            return 0
        first_key = max(0, next_pos - w + 1)
        return first_key // self.page_size

    def pages_needed(self, req_id: Hashable, new_len: int) -> List[int]:
        """New pages per group for the request to hold positions up to new_len - 1,
        given that the next step starts at its current length."""
        rc = self.get(req_id)
        need = []
        for g, table in enumerate(rc.tables):
            # entries from the first live page up to the table's end hold pages (reserve leaves
            # no holes there), so what is missing lies beyond the table's end
            lo = self._first_live_page(g, rc.num_tokens)
            hi = (new_len + self.page_size - 1) // self.page_size
            need.append(max(0, hi - max(lo, len(table))))
        return need

    def can_reserve(self, wants: Sequence[Tuple[Hashable, int]]) -> bool:
        """True if all of (request, new length) can get their pages together."""
        total = [0] * len(self.groups)
        for req_id, new_len in wants:
            for g, n in enumerate(self.pages_needed(req_id, new_len)):
                total[g] += n
        return all(total[g] <= self.available(g) for g in range(len(self.groups)))

    def available(self, group: int = 0) -> int:
        """Pages a reservation can get: the free ones and the kept ones (a kept entry has a page in every group)."""
        return self.pools[group].num_free + len(self._kept)

    @property
    def num_kept(self) -> int:
        """Registered entries that nobody holds (each has a page in every group)."""
        return len(self._kept)

    def _allocate(self, g: int) -> int:
        while not self.pools[g].free and self._kept:
            h, entry = self._kept.popitem(last=False)
            del self._shared[h]
            del self._page_hash[entry.pages[0]]
            for gg, page in enumerate(entry.pages):
                self.pools[gg].give_back(page)
                self.stats["pages_freed"] += 1
                if self.track_pages:
                    self._page_events.append((gg, page))
            self.stats["kept_pages_evicted"] += 1
        page = self.pools[g].allocate()
        if self.track_pages:
            self._page_events.append((g, page))
        return page

    def take_page_events(self) -> List[Tuple[int, int]]:
        """(group, page) of every page handed out or given back to a free list since the last call
        (only noted while ``track_pages`` is set).  Pages kept aside for a later request with the
        same prefix are not among them: their contents are still wanted."""
        out, self._page_events = self._page_events, []
        return out

    def reserve(self, req_id: Hashable, new_len: int) -> None:
        """Give the request pages for every position it will hold up to new_len - 1.
        All or nothing: raises OutOfPages and changes nothing if a pool is short."""
        rc = self.get(req_id)
        if new_len < rc.num_tokens:
            raise CacheError("a request's length cannot shrink")
        need = self.pages_needed(req_id, new_len)
        for g, n in enumerate(need):
            if n > self.available(g):
                raise OutOfPages(f"group {g} needs {n} pages for request {req_id!r}, "
                                 f"{self.available(g)} are free")
        hi = (new_len + self.page_size - 1) // self.page_size
        for g, table in enumerate(rc.tables):
            lo = self._first_live_page(g, rc.num_tokens)
            start = max(lo, len(table))
            while len(table) < start:              # behind the window from the start: never held
                table.append(-1)
            for i in range(start, hi):
                table.append(self._allocate(g))
                rc.dirty[g].append(i)
                self.stats["pages_allocated"] += 1

    def commit(self, req_id: Hashable, tokens: Sequence[int]) -> None:
        """The step has written these tokens' keys: lengthen the request, register pages
        that became full for sharing, and give back pages that a window has passed."""
        rc = self.get(req_id)
        new_len = rc.num_tokens + len(tokens)
        for g, table in enumerate(rc.tables):
            if len(table) * self.page_size < new_len:
                raise CacheError(f"request {req_id!r} has no pages reserved up to {new_len}")
        rc.tokens.extend(int(t) for t in tokens)
        rc.num_tokens = new_len
        rc.new_request = False
        if self.prefix_sharing:
            self._register_full_pages(rc)
        for g, table in enumerate(rc.tables):
            if self.groups[g].window is None:
                continue
            live_from = min(self._first_live_page(g, new_len), len(table))
            for i in range(rc.released[g], live_from):   # pages below rc.released[g] went back earlier
                if table[i] >= 0:
                    self._release(g, table[i])
                    table[i] = -1
                    rc.dirty[g].append(i)
            rc.released[g] = max(rc.released[g], live_from)

    def _release(self, g: int, page: int) -> None:
        if self.pools[g].release(page):
            self.stats["pages_freed"] += 1
            if self.track_pages:
                self._page_events.append((g, page))
            if g == 0:
                h = self._page_hash.pop(page, None)
                if h is not None:
                    self._shared.pop(h, None)

    # ---- tables and slots for a step ------------------------------------------------
    def block_table(self, req_id: Hashable, group: int) -> List[int]:
        return self.get(req_id).tables[group]

    def take_dirty(self, req_id: Hashable, group: int) -> List[Tuple[int, int]]:
        """(table index, page id) of every entry of the request's table that changed since the
        last call; for keeping a copy of the tables elsewhere (on the device) up to date."""
        rc = self.get(req_id)
        table = rc.tables[group]
        out = [(i, table[i]) for i in dict.fromkeys(rc.dirty[group])]
        rc.dirty[group] = []
        return out

    def token_slot_array(self, req_id: Hashable, group: int, start: int, count: int) -> np.ndarray:
        """page * page_size + offset for positions start .. start + count - 1, as int32."""
        table = self.get(req_id).tables[group]
        P = self.page_size
        if count <= 0:
            return np.zeros(0, dtype=np.int32)
        first, last = start // P, (start + count - 1) // P
        pages = np.asarray(table[first:last + 1], dtype=np.int64)
        if len(pages) != last + 1 - first or (pages < 0).any():
            missing = next(q for q in range(start, start + count)
                           if q // P >= len(table) or table[q // P] < 0)
            raise CacheError(f"request {req_id!r} holds no page for position {missing} in group {group}")
        pos = np.arange(start, start + count, dtype=np.int64)
        return (pages[pos // P - first] * P + pos % P).astype(np.int32)

    def token_slots(self, req_id: Hashable, group: int, start: int, count: int) -> List[int]:
        """The same as a list."""
        return self.token_slot_array(req_id, group, start, count).tolist()

    # ---- prefix sharing ----------------------------------------------------------
    def match_prefix(self, req_id: Hashable, prompt: Sequence[int]) -> int:
        """For a request that holds nothing yet: take over the pages of the longest
        registered run of full pages that equals the prompt's beginning.  At least one
        prompt token is always left to compute.  Returns the number of tokens taken over."""
        rc = self.get(req_id)
        if rc.num_tokens or any(rc.tables[g] for g in range(len(self.groups))):
            raise CacheError("a prefix can only be matched for a request that holds nothing")
        if not self.prefix_sharing:
            return 0
        P = self.page_size
        max_pages = (len(prompt) - 1) // P if prompt else 0
        parent = 0
        taken: List[_SharedEntry] = []
        hashes = []
        for i in range(max_pages):
            toks = tuple(int(t) for t in prompt[i * P:(i + 1) * P])
            h = chain_hash(parent, toks)
            entry = self._shared.get(h)
            if entry is None or entry.tokens != toks:   # the token test guards against collisions
                break
            taken.append(entry)
            hashes.append(h)
            parent = h
        for h, entry in zip(hashes, taken):
            was_kept = self._kept.pop(h, None) is not None    # held by nobody until now
            self.stats["kept_page_hits"] += int(was_kept)
            for g, page in enumerate(entry.pages):
                if was_kept:
                    self.pools[g].revive(page)
                else:
                    self.pools[g].retain(page)
                rc.dirty[g].append(len(rc.tables[g]))
                rc.tables[g].append(page)
        n = len(taken) * P
        rc.num_tokens = n
        rc.shared_len = n
        rc.tokens = [int(t) for t in prompt[:n]]
        rc.hashes = hashes
        self.stats["shared_page_hits"] += len(taken)
        return n

    def _register_full_pages(self, rc: RequestCache) -> None:
        P = self.page_size
        full = rc.num_tokens // P
        while len(rc.hashes) < full:
            i = len(rc.hashes)
            toks = tuple(rc.tokens[i * P:(i + 1) * P])
            parent = rc.hashes[-1] if rc.hashes else 0
            h = chain_hash(parent, toks)
            rc.hashes.append(h)
            pages = tuple(rc.tables[g][i] for g in range(len(self.groups)))
            if h not in self._shared and pages[0] not in self._page_hash:
                self._shared[h] = _SharedEntry(pages=pages, tokens=toks)
                self._page_hash[pages[0]] = h

    # ---- whole-manager views -------------------------------------------------------
    def num_free_pages(self, group: int = 0) -> int:
        return self.available(group)

    def reset(self) -> None:
        for req_id in list(self.requests):
            self.free_request(req_id)
        for entry in self._kept.values():
            for g, page in enumerate(entry.pages):
                self.pools[g].give_back(page)
                if self.track_pages:
                    self._page_events.append((g, page))
        self._kept.clear()
        self._shared.clear()
        self._page_hash.clear()

    def check_invariants(self) -> None:
        """No page lost, held twice without a count, or both free and held."""
        for g, pool in enumerate(self.pools):
            held: Dict[int, int] = {}
            for rc in self.requests.values():
                seen = set()
                for page in rc.tables[g]:
                    if page < 0:
                        continue
                    if page in seen:
                        raise CacheError(f"request {rc.req_id!r} holds page {page} twice in group {g}")
                    seen.add(page)
                    held[page] = held.get(page, 0) + 1
            free = set(pool.free)
            if len(free) != len(pool.free):
                raise CacheError(f"group {g}: a page is in the free list twice")
            kept = [entry.pages[g] for entry in self._kept.values()]
            if len(set(kept)) != len(kept) or free & set(kept):
                raise CacheError(f"group {g}: a page is kept twice, or kept and free")
            for page in range(pool.num_pages):
                rcnt = pool.refcount[page]
                if rcnt != held.get(page, 0):
                    raise CacheError(f"group {g}: page {page} has count {rcnt}, "
                                     f"{held.get(page, 0)} requests hold it")
                if (rcnt == 0) != (page in free or page in kept):
                    raise CacheError(f"group {g}: page {page} count {rcnt}, free: {page in free}, kept: {page in kept}")
        for h, entry in self._kept.items():
            if self._shared.get(h) is not entry:
                raise CacheError("a kept entry is not registered")
        for h, entry in self._shared.items():
            for g, page in enumerate(entry.pages):
                if (self.pools[g].refcount[page] <= 0) != (h in self._kept):
                    raise CacheError(f"registered page {page} of group {g}: held by nobody and not kept, or kept and held")
            if self._page_hash.get(entry.pages[0]) != h:
                raise CacheError("the two maps of the prefix registry disagree")
        owners = [o for o in self.slots.owner if o is not None]
        if sorted(map(repr, owners)) != sorted(map(repr, self.requests)):
            raise CacheError("state slots and live requests disagree")
