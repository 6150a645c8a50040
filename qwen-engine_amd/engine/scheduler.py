"""The scheduler: admits requests, cuts prompts into portions under a token budget,
decodes, finishes and frees.  Host logic only; it works against the cache manager's
page accounting and never touches a tensor.

The reference runs whole prompts, then one decode step, in a loop, admits without
looking at free pages and frees only when every request is done
(src/engine/llm_engine.py:101-152).  Kept from it: first in, first out; the first
new token comes from the prompt's last logits and counts toward max_new_tokens
(llm_engine.py:113-125); a request prefilled in a step decodes in the next.  New:
portions and mixed steps, a token budget, stopping on end-of-sequence tokens, release
at finish, and a rule for when pages run out:

  * a request is admitted only if its first portion's pages are free;
  * if a running request cannot get the pages for its next tokens, the request that
    was admitted last is preempted: its pages go back, it returns to the front of the
    waiting queue, and it is recomputed from its prompt and the tokens it has already
    produced when it is admitted again (sampling does not depend on that);
  * a request that cannot fit even when it has the cache to itself fails with an error.

Requests that arrive together and begin alike share their beginning too (the reference registers a
prompt's pages when it allocates them, src/engine/kvcache.py:183-195, so the prompts of one batch
find each other; here a page is registered only once it is computed): a waiting request whose
first pages equal pages that a running request is still to compute is held back until they are
computed, and then takes them over instead of computing them again.  Requests behind it in the
queue may start meanwhile.
"""
from __future__ import annotations

from collections import deque
from dataclasses import dataclass, field
from typing import Deque, Dict, Hashable, List, Optional, Sequence, Tuple

from ..cache.manager import CacheManager, chain_hash
from ..sampling.sampler import SamplingParams

WAITING, RUNNING, FINISHED = "waiting", "running", "finished"


@dataclass
class Request:
    req_id: int
    prompt: List[int]
    params: SamplingParams
    output: List[int] = field(default_factory=list)
    status: str = WAITING
    finish_reason: Optional[str] = None      # "length", "stop" or "error"
    error: Optional[str] = None
    num_computed: int = 0                    # tokens of prompt + output whose keys are cached
    admit_order: int = -1
    preemptions: int = 0
    prompt_text: Optional[str] = None
    _page_hashes: Optional[Tuple[int, int, List[int]]] = None   # (page size, tokens hashed, chain hashes)

    def page_hashes(self, page_size: int) -> List[int]:
        """Chain hashes of the full pages of the known tokens (kept; extended when tokens were added)."""
        known = self.known
        full = len(known) // page_size
        if self._page_hashes is None or self._page_hashes[0] != page_size:
            self._page_hashes = (page_size, 0, [])
        _, _, hashes = self._page_hashes
        while len(hashes) < full:
            i = len(hashes)
            hashes.append(chain_hash(hashes[-1] if hashes else 0, known[i * page_size:(i + 1) * page_size]))
        self._page_hashes = (page_size, full * page_size, hashes)
        return hashes

    @property
    def known(self) -> List[int]:
        return self.prompt + self.output

    @property
    def num_known(self) -> int:
        return len(self.prompt) + len(self.output)

    def known_span(self, start: int, n: int) -> List[int]:
        """known[start:start + n] without joining the two lists when the span lies in one of them
        (a decoding request's span is its last output token, every step)."""
        lp = len(self.prompt)
        if start >= lp:
            return self.output[start - lp:start - lp + n]
        if start + n <= lp:
            return self.prompt[start:start + n]
        return self.known[start:start + n]


@dataclass
class Planned:
    request: Request
    tokens: List[int]
    sample: bool        # the portion ends at the request's last known token: its logits give the next one


class Scheduler:
    def __init__(self, cache: CacheManager, max_num_seqs: int, max_model_len: int,
                 max_step_tokens: int, prefill_chunk: int, eos_token_ids: Sequence[int] = ()):
        self.cache = cache
        self.max_num_seqs = max_num_seqs
        self.max_model_len = max_model_len
        self.max_step_tokens = max_step_tokens
        self.prefill_chunk = prefill_chunk
        self.eos = set(int(e) for e in eos_token_ids)
        self.waiting: Deque[Request] = deque()
        self.running: List[Request] = []
        self.finished: List[Request] = []
        self._admitted = 0
        self.stats = {"steps": 0, "prefill_tokens": 0, "decode_tokens": 0, "preemptions": 0,
                      "shared_prefix_tokens": 0, "failed": 0, "held_back_for_prefix": 0}

    # ---- queue ----------------------------------------------------------------------
    def add(self, request: Request) -> None:
        request.params.validate()
        if not request.prompt:
            self._fail(request, "the prompt is empty")
            return
        if len(request.prompt) >= self.max_model_len:
            self._fail(request, f"the prompt has {len(request.prompt)} tokens, "
                                f"max_model_len is {self.max_model_len}")
            return
        self.waiting.append(request)

    def has_work(self) -> bool:
        return bool(self.waiting or self.running)

    def _fail(self, request: Request, why: str) -> None:
        request.status, request.finish_reason, request.error = FINISHED, "error", why
        self.finished.append(request)
        self.stats["failed"] += 1

    # ---- planning a step ----------------------------------------------------------------
    def _pool_pages(self) -> List[int]:
        return [p.num_pages for p in self.cache.pools]

    def _fits_alone(self, total_len: int) -> bool:
        """Could a request of this length be held if it had the cache to itself?"""
        P = self.cache.page_size
        for g, pool in enumerate(self.cache.pools):
            w = self.cache.groups[g].window
            span = total_len if w is None else min(total_len, w + self.prefill_chunk + P)
            if (span + P - 1) // P > pool.num_pages:
                return False
        return True

    def _pages_worth_waiting_for(self, r: Request, start: int) -> bool:
        """True if a running request is still to compute pages that equal r's pages beyond its first
        ``start`` tokens: r then does better to wait and take them over than to compute them itself."""
        if not self.cache.prefix_sharing:
            return False
        P = self.cache.page_size
        mine = r.page_hashes(P)[:(r.num_known - 1) // P]      # (one token is always left to compute)
        have = start // P
        if len(mine) <= have:
            return False
        for q in self.running:
            theirs = q.page_hashes(P)
            if len(theirs) <= have or theirs[have] != mine[have] or q.num_computed >= (have + 1) * P:
                continue
            # (equal chain hashes at index `have`: everything up to there is equal, up to collisions,
            # which at worst make r wait until q has computed that page)
            return True
        return False

    def _preempt_last(self) -> bool:
        """Give back the pages of the running request that was admitted last."""
        if not self.running:
            return False
        victim = max(self.running, key=lambda r: r.admit_order)
        self.cache.free_request(victim.req_id)
        self.running.remove(victim)
        victim.status = WAITING
        victim.num_computed = 0
        victim.preemptions += 1
        self.waiting.appendleft(victim)
        self.stats["preemptions"] += 1
        return True

    def plan(self) -> List[Planned]:
        """Decide the next step: decoded tokens of every running request that is ready, then
        portions of prompts, oldest first, within the token budget."""
        groups = range(len(self.cache.groups))
        while True:
            planned: List[Planned] = []
            budget = self.max_step_tokens
            blocked: Optional[Request] = None
            # The portion limit keeps a step short for the requests that decode in it.  While none
            # does, a prompt may take the whole budget: a long prompt in an idle engine then runs in
            # few large steps (8192 tokens: four steps instead of sixteen, 1.7 times sooner).
            # Several prompts at once share the budget in equal parts of at least the portion limit, so that a
            # long prompt does not hold a short one that arrived with it back until it is through.
            # What the shares leave over (a prompt shorter than its share, a request that waits for pages which
            # another is still computing) goes to the planned prompts that can use it, oldest first.
            with_prompt = sum(1 for r in self.running if r.num_known - r.num_computed > 1) + len(self.waiting)
            shares = max(1, min(with_prompt, self.max_step_tokens // self.prefill_chunk))
            decoding = any(r.num_known - r.num_computed == 1 for r in self.running)
            chunk = self.prefill_chunk if decoding else max(self.prefill_chunk, self.max_step_tokens // shares)
            # pages the entries planned so far need, per group: an entry fits if its own pages fit
            # beside them (the same answer as cache.can_reserve on the whole list, without going
            # through the list again for every candidate)
            taken = [0 for _ in groups]

            def fits(req_id, new_len) -> bool:
                need = self.cache.pages_needed(req_id, new_len)
                if any(taken[g] + need[g] > self.cache.available(g) for g in groups):
                    return False
                for g in groups:
                    taken[g] += need[g]
                return True

            for r in sorted(self.running, key=lambda r: r.admit_order):
                remaining = r.num_known - r.num_computed
                if remaining <= 0 or budget <= 0:
                    continue
                n = 1 if remaining == 1 else min(remaining, chunk, budget)
                while not fits(r.req_id, r.num_computed + n):
                    if n == 1:
                        n = 0
                        break
                    n = n // 2                                 # fewer tokens may still fit (down to one)
                if n == 0:
                    blocked = blocked or r
                    continue
                toks = r.known_span(r.num_computed, n)
                planned.append(Planned(r, toks, sample=(r.num_computed + n == r.num_known)))
                budget -= n
            if blocked is not None:
                # a running request got no pages: the newest goes back to the queue, plan again
                if len(self.running) > 1:
                    self._preempt_last()
                else:   # it holds every page that is in use, and still cannot go on
                    self.running.remove(blocked)
                    self.cache.free_request(blocked.req_id)
                    self._fail(blocked, "the cache is too small for this request")
                continue
            # admission, first in first out (a request that waits for another's pages lets the next pass)
            held: List[Request] = []
            while self.waiting and len(self.running) < self.max_num_seqs and budget > 0 \
                    and self.cache.slots.num_free > 0:
                r = self.waiting[0]
                if not self._fits_alone(min(r.num_known + 1, self.max_model_len)):
                    self.waiting.popleft()
                    self._fail(r, "the cache is too small for this request")
                    continue
                self.cache.add_request(r.req_id)
                start = self.cache.match_prefix(r.req_id, r.known)
                if self._pages_worth_waiting_for(r, start):
                    self.cache.free_request(r.req_id)
                    held.append(self.waiting.popleft())
                    self.stats["held_back_for_prefix"] += 1
                    continue
                remaining = r.num_known - start
                n = min(remaining, chunk, budget)
                least = min(remaining, self.prefill_chunk, budget)
                ok = fits(r.req_id, start + n)
                while not ok and n > least:                    # a smaller first portion may still fit
                    n = max(least, n // 2)
                    ok = fits(r.req_id, start + n)
                if not ok:
                    self.cache.free_request(r.req_id)
                    break
                self.waiting.popleft()
                r.status = RUNNING
                r.num_computed = start
                r.admit_order = self._admitted
                self._admitted += 1
                self.running.append(r)
                self.stats["shared_prefix_tokens"] += start
                planned.append(Planned(r, r.known_span(start, n), sample=(start + n == r.num_known)))
                budget -= n
            self.waiting.extendleft(reversed(held))            # back to the front, in their order
            if budget > 0 and not decoding:
                for i, p in enumerate(planned):
                    r = p.request
                    end = r.num_computed + len(p.tokens)
                    more = min(r.num_known - end, budget)
                    if more <= 0:
                        continue
                    had = self.cache.pages_needed(r.req_id, end)
                    need = self.cache.pages_needed(r.req_id, end + more)
                    if any(taken[g] + need[g] - had[g] > self.cache.available(g) for g in groups):
                        continue
                    for g in groups:
                        taken[g] += need[g] - had[g]
                    planned[i] = Planned(r, r.known_span(r.num_computed, len(p.tokens) + more),
                                         sample=(end + more == r.num_known))
                    budget -= more
            if not planned and self.waiting and not self.running:
                # nothing runs and the first waiting request cannot start: it can never start
                r = self.waiting.popleft()
                self._fail(r, "the cache is too small for this request")
                continue
            return planned

    # ---- after the step -------------------------------------------------------------------
    def update(self, planned: Sequence[Planned], sampled: Sequence[int]) -> List[Request]:
        """``sampled`` holds one token for every planned entry with ``sample``, in order."""
        done: List[Request] = []
        it = iter(sampled)
        self.stats["steps"] += 1
        for p in planned:
            r = p.request
            r.num_computed += len(p.tokens)
            if len(p.tokens) == 1 and r.num_computed > len(r.prompt):
                self.stats["decode_tokens"] += 1
            else:
                self.stats["prefill_tokens"] += len(p.tokens)
            if not p.sample:
                continue
            tok = int(next(it))
            r.output.append(tok)
            reason = None
            if tok in self.eos and not r.params.ignore_eos:
                reason = "stop"
            elif len(r.output) >= r.params.max_new_tokens:
                reason = "length"
            elif r.num_known >= self.max_model_len:
                reason = "length"
            if reason:
                r.status, r.finish_reason = FINISHED, reason
                self.running.remove(r)
                self.cache.free_request(r.req_id)
                self.finished.append(r)
                done.append(r)
        return done
