"""The scheduler's decisions (CPU), against the real cache manager and a stand-in for
the step function whose "model" makes the next token a hash of all tokens so far."""
import hashlib

import pytest

import qwen_engine_amd  # noqa: F401
from qwen_engine_amd.cache import CacheManager, GroupSpec
from qwen_engine_amd.engine.scheduler import Request, Scheduler
from qwen_engine_amd.sampling import SamplingParams


def fake_next(tokens):
    h = hashlib.blake2b(repr(list(tokens)).encode(), digest_size=4).digest()
    return int.from_bytes(h, "little") % 97 + 3          # never 0..2 (used as eos below)


def drive(sched, cache, log=None, max_steps=10_000):
    """What LLMEngine.step does, with the fake model: reserve, commit, sample, update."""
    steps = 0
    while sched.has_work():
        planned = sched.plan()
        if not planned:
            break
        assert len({p.request.req_id for p in planned}) == len(planned)
        assert sum(len(p.tokens) for p in planned) <= sched.max_step_tokens
        assert cache.can_reserve([(p.request.req_id, p.request.num_computed + len(p.tokens)) for p in planned])
        sampled = []
        for p in planned:
            r = p.request
            assert p.tokens == r.known[r.num_computed:r.num_computed + len(p.tokens)]
            assert cache.get(r.req_id).num_tokens == r.num_computed
            cache.reserve(r.req_id, r.num_computed + len(p.tokens))
            cache.commit(r.req_id, p.tokens)
            if p.sample:
                sampled.append(fake_next(r.known))
        if log is not None:
            log.append([(p.request.req_id, len(p.tokens), p.sample) for p in planned])
        sched.update(planned, sampled)
        cache.check_invariants()
        steps += 1
        assert steps < max_steps
    return steps


def make(num_pages=64, page=4, max_num_seqs=4, max_model_len=256, budget=64, chunk=16, eos=(), sharing=False):
    cache = CacheManager([GroupSpec()], num_pages, page_size=page, max_requests=max_num_seqs, prefix_sharing=sharing)
    return Scheduler(cache, max_num_seqs, max_model_len, budget, chunk, eos), cache


def expected_output(prompt, n):
    toks, out = list(prompt), []
    for _ in range(n):
        t = fake_next(toks)
        out.append(t)
        toks.append(t)
    return out


PROMPTS = [[5, 6, 7, 8, 9], list(range(10, 19)), list(range(20, 33)), [40] * 30]


def test_every_request_gets_exactly_its_tokens():
    sched, cache = make()
    reqs = [Request(i, p, SamplingParams(max_new_tokens=8)) for i, p in enumerate(PROMPTS)]
    for r in reqs:
        sched.add(r)
    drive(sched, cache)
    for r in reqs:
        assert r.finish_reason == "length" and r.output == expected_output(r.prompt, 8)
    assert all(pool.num_free == pool.num_pages for pool in cache.pools)      # freed at finish
    assert cache.slots.num_free == 4


def test_outputs_do_not_depend_on_sizes_of_the_engine():
    want = [expected_output(p, 10) for p in PROMPTS]
    for kw in (dict(max_num_seqs=1), dict(budget=3, chunk=2), dict(budget=7, chunk=6), dict(num_pages=14),
               dict(page=1, num_pages=60), dict(sharing=True), dict(num_pages=11, budget=5, chunk=4)):
        sched, cache = make(**kw)
        reqs = [Request(i, p, SamplingParams(max_new_tokens=10)) for i, p in enumerate(PROMPTS)]
        for r in reqs:
            sched.add(r)
        drive(sched, cache)
        assert [r.output for r in reqs] == want, kw
        assert all(pool.num_free == pool.num_pages for pool in cache.pools)


def test_prompts_are_cut_under_the_budget_and_mixed_with_decodes():
    sched, cache = make(budget=8, chunk=6)
    a = Request(0, list(range(3, 8)), SamplingParams(max_new_tokens=6))
    b = Request(1, list(range(30, 50)), SamplingParams(max_new_tokens=2))
    sched.add(a)
    sched.add(b)
    log = []
    drive(sched, cache, log)
    # step 0: a's whole prompt (5), then b's first portion cut to the 3 tokens that are left
    assert log[0] == [(0, 5, True), (1, 3, False)]
    # step 1: a decodes one token beside b's next portion of 6 (the chunk size)
    assert log[1] == [(0, 1, True), (1, 6, False)]
    assert log[2] == [(0, 1, True), (1, 6, False)]
    assert log[3] == [(0, 1, True), (1, 5, True)]        # b's last portion gives its first token
    assert all(sum(n for _, n, _ in step) <= 8 for step in log)


def test_a_prompt_takes_the_whole_budget_while_nothing_decodes():
    """The portion limit protects the requests that decode: an idle engine runs a long prompt in steps
    of the whole budget, and goes back to the limit as soon as a request decodes beside it."""
    sched, cache = make(num_pages=200, budget=32, chunk=8, max_model_len=400)
    a = Request(0, list(range(3, 103)), SamplingParams(max_new_tokens=3))          # 100 tokens
    sched.add(a)
    log = []
    drive(sched, cache, log)
    assert [step for step in log[:4]] == [[(0, 32, False)], [(0, 32, False)], [(0, 32, False)], [(0, 4, True)]]
    assert a.output == expected_output(a.prompt, 3)
    # a short request decodes while a long prompt arrives: the long one goes in portions of the limit
    sched, cache = make(num_pages=200, budget=32, chunk=8, max_model_len=400)
    short = Request(1, [5, 6, 7], SamplingParams(max_new_tokens=20))
    long = Request(2, list(range(3, 63)), SamplingParams(max_new_tokens=2))         # 60 tokens
    sched.add(short)
    log = []
    planned = sched.plan()
    assert [(p.request.req_id, len(p.tokens)) for p in planned] == [(1, 3)]
    sampled = []
    for p in planned:
        cache.reserve(p.request.req_id, len(p.tokens)); cache.commit(p.request.req_id, p.tokens)
        sampled.append(fake_next(p.request.known))
    sched.update(planned, sampled)
    sched.add(long)
    drive(sched, cache, log)
    portions = [n for step in log for rid, n, _ in step if rid == 2 and n > 1]
    assert portions[:7] == [8] * 7 and portions[7] == 4            # while request 1 decodes beside it
    assert short.output == expected_output(short.prompt, 20) and long.output == expected_output(long.prompt, 2)


def test_prompts_that_arrive_together_share_the_budget():
    """A long and a short prompt arrive in an idle engine: the long one does not take the whole budget step
    after step; the short one's first token comes from the first step."""
    sched, cache = make(num_pages=200, budget=32, chunk=8, max_model_len=400)
    long = Request(0, list(range(3, 103)), SamplingParams(max_new_tokens=2))        # 100 tokens
    short = Request(1, [5, 6, 7, 8, 9], SamplingParams(max_new_tokens=2))
    sched.add(long)
    sched.add(short)
    log = []
    drive(sched, cache, log)
    # two prompts: half the budget each; what the short one leaves of its half goes to the long one
    assert log[0] == [(0, 16 + 11, False), (1, 5, True)]
    assert log[1][0] == (0, 8, False)                          # the short one decodes now: portions of the limit
    assert long.output == expected_output(long.prompt, 2) and short.output == expected_output(short.prompt, 2)
    # three prompts and a budget of four portions: a third of the budget each, rounded down, at least a portion
    sched, cache = make(num_pages=400, budget=32, chunk=8, max_model_len=400, max_num_seqs=4)
    for i in range(3):
        sched.add(Request(i, list(range(3, 103)), SamplingParams(max_new_tokens=1)))
    planned = sched.plan()
    assert [(p.request.req_id, len(p.tokens)) for p in planned] == [(0, 10 + 2), (1, 10), (2, 10)]
    # requests that wait for pages which the first is still computing take no share: the first gets the budget
    common = list(range(3, 43))
    sched, cache = make(num_pages=400, budget=32, chunk=8, max_model_len=400, max_num_seqs=4, sharing=True)
    for i in range(4):
        sched.add(Request(i, common + [50 + i], SamplingParams(max_new_tokens=1)))
    planned = sched.plan()
    assert [(p.request.req_id, len(p.tokens)) for p in planned] == [(0, 32)]
    assert sched.stats["held_back_for_prefix"] == 3
    # a top-up that has no pages is left out: 10 pages of 4 tokens, two prompts of 36 and shares of 24 (the
    # second's made smaller until it fits: 6 + 3 pages), 12 tokens of the budget left and one page
    sched, cache = make(num_pages=10, budget=48, chunk=8, max_model_len=64, max_num_seqs=2)
    for i in range(2):
        sched.add(Request(i, list(range(3, 39)), SamplingParams(max_new_tokens=1)))
    planned = sched.plan()
    assert [(p.request.req_id, len(p.tokens)) for p in planned] == [(0, 24), (1, 12)]
    assert cache.can_reserve([(p.request.req_id, p.request.num_computed + len(p.tokens)) for p in planned])


def test_a_first_portion_of_the_whole_budget_that_does_not_fit_is_made_smaller():
    """12 pages of 4 tokens: a prompt of 40 tokens cannot take a first portion of the whole budget (64
    tokens would be the limit, 40 tokens are 10 pages, and 5 pages are held by another request), but a
    smaller one fits: it is admitted with that instead of waiting or failing."""
    sched, cache = make(num_pages=12, page=4, budget=64, chunk=8, max_model_len=64, max_num_seqs=2)
    cache.add_request("other")
    cache.reserve("other", 20)
    cache.commit("other", list(range(20)))
    r = Request(0, list(range(3, 43)), SamplingParams(max_new_tokens=1))
    sched.add(r)
    planned = sched.plan()
    assert [(p.request.req_id, len(p.tokens)) for p in planned] == [(0, 20)]       # 40 -> 20 tokens: 5 pages fit beside the 5
    assert r.status != "failed"


def test_admission_is_first_in_first_out_and_bounded():
    sched, cache = make(max_num_seqs=2)
    reqs = [Request(i, [7 + i] * 6, SamplingParams(max_new_tokens=3)) for i in range(5)]
    for r in reqs:
        sched.add(r)
    log = []
    drive(sched, cache, log)
    first_seen = {}
    for s, step in enumerate(log):
        assert len(step) <= 2
        for rid, _, _ in step:
            first_seen.setdefault(rid, s)
    assert [first_seen[i] for i in range(5)] == sorted(first_seen[i] for i in range(5))


def test_stops_on_eos_unless_told_not_to():
    prompt = [5, 6, 7]
    out = expected_output(prompt, 12)
    eos = out[4]
    first = out.index(eos)
    sched, cache = make(eos=(eos,))
    r = Request(0, prompt, SamplingParams(max_new_tokens=12))
    r2 = Request(1, prompt, SamplingParams(max_new_tokens=12, ignore_eos=True))
    sched.add(r)
    sched.add(r2)
    drive(sched, cache)
    assert r.finish_reason == "stop" and r.output == out[:first + 1]
    assert r2.finish_reason == "length" and r2.output == out


def test_length_is_capped_by_max_model_len():
    sched, cache = make(max_model_len=12)
    r = Request(0, list(range(3, 11)), SamplingParams(max_new_tokens=50))
    sched.add(r)
    drive(sched, cache)
    assert r.finish_reason == "length" and len(r.prompt) + len(r.output) == 12
    too_long = Request(1, [4] * 12, SamplingParams())
    sched.add(too_long)
    assert too_long.finish_reason == "error" and "max_model_len" in too_long.error


def test_when_pages_run_out_the_newest_request_is_preempted_and_recomputed():
    # 3 requests of 8 + 12 tokens need 5 pages each at the end; 9 pages cannot hold them all
    sched, cache = make(num_pages=9, page=4, max_num_seqs=3)
    reqs = [Request(i, [11 * (i + 1)] * 8, SamplingParams(max_new_tokens=12)) for i in range(3)]
    for r in reqs:
        sched.add(r)
    drive(sched, cache)
    assert sched.stats["preemptions"] > 0
    assert reqs[0].preemptions == 0                      # the oldest is never the victim
    for r in reqs:
        assert r.finish_reason == "length" and r.output == expected_output(r.prompt, 12)
    assert all(pool.num_free == pool.num_pages for pool in cache.pools)


def test_a_request_that_can_never_fit_fails_alone():
    sched, cache = make(num_pages=3, page=4)
    big = Request(0, [9] * 20, SamplingParams(max_new_tokens=2))      # 6 pages > 3
    small = Request(1, [8] * 5, SamplingParams(max_new_tokens=2))
    grows = Request(2, [7] * 10, SamplingParams(max_new_tokens=30))   # fits at first, then outgrows the pool
    for r in (big, small, grows):
        sched.add(r)
    drive(sched, cache)
    assert big.finish_reason == "error" and "cache is too small" in big.error
    assert small.finish_reason == "length" and small.output == expected_output(small.prompt, 2)
    assert grows.finish_reason == "error" and grows.output == expected_output(grows.prompt, len(grows.output))
    assert all(pool.num_free == pool.num_pages for pool in cache.pools)


def test_shared_prefix_is_taken_over_at_admission():
    sched, cache = make(page=4, sharing=True, max_num_seqs=2, budget=64, chunk=64)
    common = list(range(50, 66))                          # 16 tokens = 4 pages
    a = Request(0, common + [1, 2, 3], SamplingParams(max_new_tokens=4))
    b = Request(1, common + [4, 5], SamplingParams(max_new_tokens=4))
    sched.add(a)
    log = []
    planned = sched.plan()
    for p in planned:
        cache.reserve(p.request.req_id, p.request.num_computed + len(p.tokens))
        cache.commit(p.request.req_id, p.tokens)
    sched.update(planned, [fake_next(a.known)])
    sched.add(b)
    drive(sched, cache, log)
    assert (1, 2, True) in log[0]                         # b computes only its own two tokens
    assert sched.stats["shared_prefix_tokens"] == 16
    assert a.output == expected_output(a.prompt, 4) and b.output == expected_output(b.prompt, 4)


def test_bad_requests_are_refused():
    sched, _ = make()
    r = Request(0, [], SamplingParams())
    sched.add(r)
    assert r.finish_reason == "error"
    with pytest.raises(ValueError):
        sched.add(Request(1, [1], SamplingParams(max_new_tokens=0)))
    with pytest.raises(ValueError):
        sched.add(Request(2, [1], SamplingParams(temperature=-1.0)))


def test_requests_that_arrive_together_share_their_beginning():
    """The reference's prompt pair (main.py:64-68: the third prompt is the beginning of the second),
    submitted in one batch: the second of the pair waits until the first has computed the pages
    they have in common and takes them over, a request between them that shares nothing starts
    at once, and the tokens are the same as without sharing."""
    common = [50 + (7 * i) % 40 for i in range(22)]          # five full pages of four tokens and a half
    prompts = [common + [91, 92, 93, 94, 95, 96], common[:20], [3, 1, 4, 1, 5, 9, 2, 6], common + [77]]
    want = [expected_output(p, 6) for p in prompts]
    for chunk in (8, 64):
        sched, cache = make(sharing=True, chunk=chunk, budget=64)
        reqs = [Request(i, p, SamplingParams(max_new_tokens=6)) for i, p in enumerate(prompts)]
        for r in reqs:
            sched.add(r)
        log = []
        drive(sched, cache, log)
        assert [r.output for r in reqs] == want
        first = [rid for rid, _, _ in log[0]]
        assert first == [0, 2]                                # 1 and 3 wait for request 0's pages; 2 passes them
        # request 1 (20 tokens = 5 pages, one token always left: 4 pages taken over), request 3 (5 pages)
        assert sched.stats["shared_prefix_tokens"] == 16 + 20
        assert sched.stats["held_back_for_prefix"] >= 2
        n_prefill = sum(n for step in log for _, n, _ in step) - sched.stats["decode_tokens"]
        assert n_prefill == sum(len(p) for p in prompts) - 36
    # without sharing nothing waits
    sched, cache = make(sharing=False)
    for i, p in enumerate(prompts):
        sched.add(Request(i, p, SamplingParams(max_new_tokens=6)))
    log = []
    drive(sched, cache, log)
    assert [rid for rid, _, _ in log[0]] == [0, 1, 2, 3] and sched.stats["held_back_for_prefix"] == 0


def test_a_request_held_back_for_a_prefix_goes_on_when_the_other_is_preempted_or_ends():
    """The running request that the pages were expected from is preempted (too few pages) or ends
    before it has computed them: the one that waited computes its prompt itself."""
    common = list(range(30, 46))
    a, b = common + [1, 2, 3], common + [4, 5]
    sched, cache = make(num_pages=7, sharing=True, chunk=4, budget=8, max_num_seqs=2)
    ra, rb = Request(0, a, SamplingParams(max_new_tokens=3)), Request(1, b, SamplingParams(max_new_tokens=3))
    sched.add(ra)
    sched.add(rb)
    drive(sched, cache)
    assert ra.output == expected_output(a, 3) and rb.output == expected_output(b, 3)
    assert ra.finish_reason == rb.finish_reason == "length"
    assert all(pool.num_free + cache.num_kept == pool.num_pages for pool in cache.pools)
