"""The scheduler's decisions on the CPU, with a stand-in for the model (the next token is a function
of the tokens so far, so recomputation after an eviction must give the same continuation)."""
import random

import pytest

from ginfer_amd.cache import CacheManager, OutOfPages
from ginfer_amd.engine.scheduler import Scheduler
from ginfer_amd.engine.sequence import Sequence, State
from ginfer_amd.parts import KVCacheSpec
from ginfer_amd.sampling import SamplingParams, uniform


def make(num_pages, page_size=4, max_num_seqs=4, budget=16, eos=(999,), max_model_len=256, window=None,
         prefix_caching=False):
    cache = CacheManager([KVCacheSpec(1, 16, window)], page_size, num_pages, max_num_seqs, prefix_caching=prefix_caching)
    return Scheduler(cache, max_num_seqs, budget, eos, max_model_len), cache


def fake_token(ids):
    return (sum(ids) * 31 + len(ids)) % 900


def run(sched, cache, seqs, check=None, max_steps=10000):
    for s in seqs:
        sched.add(s)
    done, steps = [], []
    while not sched.is_finished():
        batch = sched.schedule()
        assert batch, "an empty step"
        assert sum(b.num_tokens for b in batch) <= sched.max_num_batched_tokens
        assert len({id(b.seq) for b in batch}) == len(batch)
        cache.check()
        toks = []
        for b in batch:
            assert cache.pending(b.seq.request_id) == b.num_tokens
            assert cache.length(b.seq.request_id) == b.seq.num_computed
            assert b.samples == (b.seq.num_computed + b.num_tokens == b.seq.num_tokens)
            if b.samples:
                toks.append(fake_token(b.seq.token_ids))
        if check:
            check(batch)
        steps.append([(b.seq.request_id, b.num_tokens) for b in batch])
        done += sched.postprocess(batch, toks, now=float(len(steps)))
        cache.check()
        assert len(steps) < max_steps
    return done, steps


def seq(i, prompt_len, max_tokens=8, **kw):
    return Sequence(i, [(i * 7 + j) % 900 for j in range(prompt_len)], prompt_len, SamplingParams(max_tokens=max_tokens, **kw))


def expected(s0):
    ids = list(s0.token_ids[:s0.num_prompt_tokens])
    for _ in range(s0.params.max_tokens):
        ids.append(fake_token(ids))
    return ids


def test_prompts_are_cut_under_the_budget_and_decoding_goes_on_beside_them():
    sched, cache = make(num_pages=64, budget=16)
    a, b = seq(0, 5, max_tokens=12), seq(1, 40, max_tokens=4)
    done, steps = run(sched, cache, [a, b])
    assert steps[0] == [(0, 5), (1, 11)]                       # arrival order, the second prompt cut to the budget
    assert steps[1] == [(0, 1), (1, 15)]                       # a decoded token beside a portion
    assert steps[2] == [(0, 1), (1, 14)]                       # the prompt ends: this portion samples
    assert steps[3] == [(0, 1), (1, 1)]
    assert {s.request_id: s.token_ids for s in done} == {0: expected(a), 1: expected(b)}
    assert all(s.finish_reason == "max_tokens" for s in done) and not cache.requests


def test_admission_is_in_arrival_order_and_bounded():
    sched, cache = make(num_pages=64, max_num_seqs=2, budget=64)
    seqs = [seq(i, 6, max_tokens=3) for i in range(5)]
    done, steps = run(sched, cache, seqs)
    assert steps[0] == [(0, 6), (1, 6)]                        # two at a time
    assert all(len(st) <= 2 for st in steps)
    assert [s.request_id for s in done] == [0, 1, 2, 3, 4]
    first_step = {}
    for i, st in enumerate(steps):
        for rid, _ in st:
            first_step.setdefault(rid, i)
    assert [first_step[i] for i in range(5)] == sorted(first_step[i] for i in range(5))


def test_finishing_rules():
    sched, cache = make(num_pages=64)
    a = seq(0, 4, max_tokens=50)
    stop_tok = expected(a)[4 + 2]
    a.params.stop_token_ids = [stop_tok]
    b = seq(1, 4, max_tokens=50, ignore_eos=True)
    b.params.stop_token_ids = [expected(b)[4]]
    c = seq(2, 250, max_tokens=50)
    sched.max_num_batched_tokens = 300
    done, _ = run(sched, cache, [a, b, c])
    by = {s.request_id: s for s in done}
    assert by[0].finish_reason == "eos" and by[0].num_output_tokens == 3 and by[0].token_ids[-1] == stop_tok
    assert by[1].finish_reason == "max_tokens" and by[1].num_output_tokens == 50
    assert by[2].finish_reason == "max_model_len" and by[2].num_tokens == 256
    # the configuration's ids apply when the request names none
    sched2, cache2 = make(num_pages=64, eos=(expected(seq(0, 4))[5],))
    d = seq(0, 4, max_tokens=50)
    done, _ = run(sched2, cache2, [d])
    assert done[0].finish_reason == "eos" and done[0].num_output_tokens == 2


def test_out_of_pages_evicts_the_newest_and_recomputes_it():
    # 3 requests of 10 + up to 14 tokens: 24 tokens = 6 pages each; 12 pages hold two of them
    sched, cache = make(num_pages=12, budget=32)
    seqs = [seq(i, 10, max_tokens=14) for i in range(3)]
    evicted = []
    real_evict = sched._evict
    def spy(s):
        evicted.append((s.request_id, [r.request_id for r in sched.running]))
        real_evict(s)
    sched._evict = spy
    done, steps = run(sched, cache, seqs)
    assert evicted, "the pool was large enough: nothing was evicted"
    for victim, running in evicted:
        assert victim == running[-1]                            # the newest running request goes
    assert sched.num_evictions == len(evicted)
    # recomputation feeds prompt and output again and continues where it stopped
    assert {s.request_id: s.token_ids for s in done} == {i: expected(seqs[i]) for i in range(3)}
    assert max(s.evictions for s in done) >= 1 and done[0].request_id == 0
    assert not cache.requests and cache.groups[0].pool.num_free == 12


def test_a_request_that_could_never_fit_is_refused():
    sched, cache = make(num_pages=4, page_size=4)
    with pytest.raises(ValueError, match="could never finish"):
        sched.add(seq(0, 10, max_tokens=10))
    sched.add(seq(1, 10, max_tokens=6))                        # 16 tokens: exactly the pool
    with pytest.raises(ValueError, match="empty prompt"):
        sched.add(Sequence(2, [], 0, SamplingParams()))
    with pytest.raises(ValueError, match="max_model_len"):
        sched.add(seq(3, 256))


def test_lone_request_fills_the_pool_and_finishes():
    sched, cache = make(num_pages=4, page_size=4, budget=5)
    a = seq(0, 10, max_tokens=6)
    done, steps = run(sched, cache, [a])
    assert steps[:2] == [[(0, 5)], [(0, 5)]] and done[0].token_ids == expected(a)


def test_portions_shrink_to_the_free_pages():
    sched, cache = make(num_pages=8, page_size=4, budget=64, max_num_seqs=3)
    a, b = seq(0, 20, max_tokens=4), seq(1, 30, max_tokens=2)
    done, steps = run(sched, cache, [a, b])
    assert steps[0] == [(0, 20), (1, 12)]                      # 5 pages for a, the 3 left hold 12 tokens of b
    assert {s.request_id: s.token_ids for s in done} == {0: expected(a), 1: expected(b)}


@pytest.mark.parametrize("seed", range(6))
def test_random_workloads_finish_with_the_same_tokens(seed):
    rng = random.Random(seed)
    window = rng.choice([None, 12])
    sched, cache = make(num_pages=rng.choice([16, 24, 40]), page_size=rng.choice([4, 8]), max_num_seqs=rng.choice([2, 4]),
                        budget=rng.choice([8, 24, 64]), window=window)
    cap = min(g.pool.num_pages for g in cache.groups) * cache.page_size
    seqs = []
    for i in range(12):
        n = rng.randint(1, min(40, cap - 12))
        seqs.append(seq(i, n, max_tokens=rng.randint(1, 12)))
    done, steps = run(sched, cache, seqs)
    assert {s.request_id: s.token_ids for s in done} == {s.request_id: expected(s) for s in seqs}
    assert not cache.requests and all(g.pool.num_free == g.pool.num_pages for g in cache.groups)


def test_uniform_numbers_are_a_function_of_seed_and_place():
    us = [uniform(3, n) for n in range(1000)]
    assert all(0.0 <= u < 1.0 for u in us) and len(set(us)) > 990
    assert us == [uniform(3, n) for n in range(1000)] and uniform(4, 0) != uniform(3, 0)
    # a request that names no seed draws from a stream of its own: a function of its id, different for every request
    from ginfer_amd.sampling import request_seed
    seeds = [request_seed(i) for i in range(1000)]
    assert len(set(seeds)) == 1000 and seeds == [request_seed(i) for i in range(1000)]
    assert SamplingParams().seed is None
    assert abs(sum(us) / 1000 - 0.5) < 0.05
    import numpy as np
    assert all(float(np.float32(u)) == u for u in us)          # exact in 32-bit


def run_ahead(sched, cache, seqs, arrivals=None, max_steps=10000):
    """As the engine drives the scheduler when it launches decode steps ahead: a step is advanced at once, the
    step after it is reserved (if schedule_ahead allows) before the first one's tokens are absorbed.  The
    stand-in model can name a token only once the tokens before it are known, so tokens of a step launched ahead
    are worked out when they are absorbed."""
    for s in seqs:
        sched.add(s)
    done, launched, ahead_steps, steps = [], None, 0, 0
    while launched is not None or not sched.is_finished():
        cur = launched
        if cur is None:
            cur = sched.schedule()
            assert cur
            sched.advance(cur)
        nxt = sched.schedule_ahead(cur)
        if nxt is not None:
            items, index = nxt
            assert [cur[i].seq for i in index] == [sc.seq for sc in items]
            assert all(cache.pending(sc.seq.request_id) == 1 for sc in items)
            sched.advance(items)
            ahead_steps += 1
        toks = [fake_token(b.seq.token_ids) for b in cur if b.samples]
        done += sched.absorb(cur, toks, now=float(steps))
        cache.check()
        launched = None if nxt is None else nxt[0]
        steps += 1
        if arrivals and steps in arrivals:
            sched.add(arrivals[steps])
        assert steps < max_steps
    return done, ahead_steps


def test_steps_launched_ahead_give_the_same_tokens():
    sched, cache = make(num_pages=64, max_num_seqs=3, budget=16)
    seqs = [seq(0, 5, 9), seq(1, 11, 4), seq(2, 3, 12), seq(3, 7, 6)]
    want = {s.request_id: expected(s) for s in seqs}
    done, ahead = run_ahead(sched, cache, seqs)
    assert ahead > 5
    assert {s.request_id: s.token_ids for s in done} == want
    assert not cache.requests


def test_a_request_that_stops_on_an_unseen_token_runs_one_step_too_many_and_is_dropped():
    sched, cache = make(num_pages=64, max_num_seqs=2, budget=16)
    a, b = seq(0, 4, 20), seq(1, 6, 20)
    stop = expected(a)[4 + 3]                                    # a's fourth output token ends it
    a.params.stop_token_ids = [stop]
    a.params.ignore_eos = False
    done, ahead = run_ahead(sched, cache, [a, b])
    by_id = {s.request_id: s for s in done}
    assert by_id[0].finish_reason == "eos" and by_id[0].token_ids[-1] == stop and by_id[0].num_output_tokens <= 4
    assert by_id[1].token_ids == expected(b) and by_id[1].finish_reason == "max_tokens"
    assert ahead > 5 and not cache.requests


def test_no_step_ahead_when_the_next_step_is_not_certain():
    sched, cache = make(num_pages=64, max_num_seqs=2, budget=16)
    a = seq(0, 4, 2)
    sched.add(a)
    first = sched.schedule()
    sched.advance(first)
    assert sched.schedule_ahead(first) is not None               # token 1 of 2 is on its way: one more step is certain
    cache.requests[0].pending = 0                                # (undo the reservation of the probe)
    sched.absorb(first, [fake_token(a.token_ids)], 0.0)
    second = sched.schedule()
    sched.advance(second)
    assert sched.schedule_ahead(second) is None                  # the token on its way is the last: max_tokens
    sched.absorb(second, [fake_token(a.token_ids)], 1.0)
    assert sched.is_finished()
    # a waiting request that could be admitted goes first
    sched, cache = make(num_pages=64, max_num_seqs=2, budget=16)
    sched.add(seq(0, 4, 9))
    first = sched.schedule()
    sched.advance(first)
    sched.add(seq(1, 4, 9))
    assert sched.schedule_ahead(first) is None
    # a prompt that is not through yet
    sched, cache = make(num_pages=64, max_num_seqs=2, budget=4)
    sched.add(seq(0, 9, 9))
    first = sched.schedule()
    sched.advance(first)
    assert not first[0].samples and sched.schedule_ahead(first) is None


def test_no_step_ahead_without_pages_and_nothing_stays_reserved():
    """Two requests that outgrow the pool together: where the step ahead lacks a page it is not taken, what it had
    reserved is undone, and the ordinary schedule (which may evict) decides instead; the tokens stay the same."""
    sched, cache = make(num_pages=5, page_size=4, max_num_seqs=2, budget=16)
    seqs = [seq(0, 4, 9), seq(1, 4, 9)]
    want = {s.request_id: expected(s) for s in seqs}
    for s in seqs:
        sched.add(s)
    refused_for_pages, done, steps = 0, [], 0
    while not sched.is_finished():
        batch = sched.schedule()
        sched.advance(batch)
        free_before = cache.groups[0].pool.num_free
        ahead = sched.schedule_ahead(batch)
        if ahead is None:
            assert all(r.pending == 0 for r in cache.requests.values())
            if len(batch) == 2 and all(b.samples for b in batch) and free_before < 2 \
                    and all(cache.length(b.seq.request_id) % 4 == 0 for b in batch):
                refused_for_pages += 1
        else:                                       # this test drives the steps one by one: give the probe back
            for sc in ahead[0]:
                cache.requests[sc.seq.request_id].pending = 0
        cache.check()
        done += sched.absorb(batch, [fake_token(b.seq.token_ids) for b in batch if b.samples], float(steps))
        steps += 1
        assert steps < 200
    assert refused_for_pages >= 1 and sched.num_evictions >= 1
    assert {s.request_id: s.token_ids for s in done} == want


# ---- requests that share a prefix

def test_a_request_starts_behind_the_prefix_that_the_cache_holds():
    sched, cache = make(num_pages=16, budget=32, prefix_caching=True)
    a = seq(0, 10, max_tokens=3)
    done, steps = run(sched, cache, [a])
    assert steps[0] == [(0, 10)] and done[0].token_ids == expected(a)
    # the same prompt with another end: two pages of four are known, the rest runs
    b = Sequence(1, a.token_ids[:9] + [5, 6, 7], 12, SamplingParams(max_tokens=3))
    # the whole of a's prompt and output again: everything up to the last full page is known
    c = Sequence(2, list(a.token_ids), len(a.token_ids), SamplingParams(max_tokens=2))
    done, steps = run(sched, cache, [b, c])
    assert steps[0] == [(1, 4), (2, 1)]
    assert cache.prefix_hit_tokens == 8 + 12
    assert {s.request_id: s.token_ids for s in done} == {1: expected(b), 2: expected(c)}
    assert all(g.pool.num_free == g.pool.num_pages for g in cache.groups)


def test_a_sharer_that_waits_for_pages_counts_its_hit_once():
    """8 pages of 8: a request of 56 tokens decodes and holds 7 pages (8 once it crosses a page's edge); a second one
    shares its first 32 tokens and has to wait, admitted and sent back step after step, until pages are free.  The
    tokens found in the cache count once, when its first portion is reserved."""
    sched, cache = make(num_pages=8, page_size=8, budget=64, max_num_seqs=2, prefix_caching=True)
    a = seq(0, 56, max_tokens=6)
    b = Sequence(1, a.token_ids[:32] + [3] * 12, 44, SamplingParams(max_tokens=2))
    waited, first_portion = [], []

    def on_admit(step, batch, hits):
        if b.state is State.WAITING and step >= 2:
            waited.append(step)
            assert cache.prefix_hit_tokens == 0 and hits == 0
        for sc in batch:
            if sc.seq is b and not first_portion:
                first_portion.append((step, sc.num_tokens, hits))
    done = run_as_the_engine(sched, cache, [a], arrivals={2: b}, on_admit=on_admit)
    assert len(waited) >= 3, "the second request did not have to wait: %s" % waited
    assert first_portion and first_portion[0][2] == 32       # the hit is booked with the first portion, 32 tokens
    assert cache.prefix_hit_tokens == 32
    assert {s.request_id: s.token_ids for s in done} == {0: expected(a), 1: expected(b)}
    assert all(g.pool.num_free == g.pool.num_pages for g in cache.groups)


def run_as_the_engine(sched, cache, seqs, arrivals=None, on_admit=None, max_steps=10000):
    """The engine's own order of calls around a step, without the device: schedule (which reserves), the runner's
    bookkeeping for the step's entries (which finds everything reserved and so commits nothing), advance (which commits
    with the requests' tokens), then the tokens are absorbed.  arrivals: {step number: sequence added before that step}."""
    from ginfer_amd.engine.runner import reserve_for_step, StepEntry
    for s in seqs:
        sched.add(s)
    done, steps = [], 0
    while not sched.is_finished() or (arrivals and any(k >= steps for k in arrivals)):
        if arrivals and steps in arrivals:
            sched.add(arrivals[steps])
        hits_before = cache.prefix_hit_tokens
        batch = sched.schedule()
        if on_admit:
            on_admit(steps, batch, cache.prefix_hit_tokens - hits_before)
        entries = [StepEntry(b.seq.request_id, b.seq.token_ids[b.seq.num_computed:b.seq.num_computed + b.num_tokens], [])
                   for b in batch]
        reserved = []
        reserve_for_step(cache, entries, sched.max_model_len, reserved)
        assert reserved == []                    # the scheduler had reserved every token
        for rid in reserved:
            cache.commit(rid)
        sched.advance(batch)
        cache.check()
        done += sched.absorb(batch, [fake_token(b.seq.token_ids) for b in batch if b.samples], now=float(steps))
        cache.check()
        steps += 1
        assert steps < max_steps
    return done


@pytest.mark.parametrize("finished_first", [False, True])
def test_a_request_finds_the_pages_of_a_request_that_is_still_running(finished_first):
    """Pages are remembered as soon as they are full and committed (ginfer/engine/block_manager.cc:98-108), not when
    their request ends: a request that arrives while the first one still decodes starts behind the 48 tokens that
    the two have in common."""
    sched, cache = make(num_pages=64, page_size=8, budget=64, prefix_caching=True)
    a = seq(0, 50, max_tokens=3 if finished_first else 30)
    b = Sequence(1, a.token_ids[:48] + [901, 902, 903], 51, SamplingParams(max_tokens=4))
    seen = {}

    def on_admit(step, batch, hits):
        for sc in batch:
            if sc.seq is b and b.request_id not in seen:
                seen[b.request_id] = (hits, sc.seq.num_computed, sc.num_tokens, a.state)
    done = run_as_the_engine(sched, cache, [a], arrivals={6: b}, on_admit=on_admit)
    hits, behind, ran, state_of_a = seen[1]
    assert (hits, behind, ran) == (48, 48, 3)
    assert state_of_a is (State.FINISHED if finished_first else State.RUNNING)
    assert {s.request_id: s.token_ids for s in done} == {0: expected(a), 1: expected(b)}
    # without sharing nothing is found
    sched, cache = make(num_pages=64, page_size=8, budget=64, prefix_caching=False)
    a = seq(0, 50, max_tokens=30)
    b = Sequence(1, a.token_ids[:48] + [901, 902, 903], 51, SamplingParams(max_tokens=4))
    seen.clear()
    run_as_the_engine(sched, cache, [a], arrivals={6: b}, on_admit=on_admit)
    assert seen[1][:3] == (0, 0, 51)


def test_an_evicted_request_finds_its_own_pages_again():
    sched, cache = make(num_pages=8, page_size=4, max_num_seqs=2, budget=32, prefix_caching=True)
    a, b = seq(0, 9, max_tokens=12), seq(1, 9, max_tokens=12)
    fed_again = []

    def check(batch):
        for sc in batch:
            if sc.seq is b and sc.seq.evictions and sc.num_tokens > 1:
                fed_again.append((sc.seq.num_computed, sc.num_tokens))

    done, steps = run(sched, cache, [a, b], check=check)
    assert b.evictions == 1 and a.evictions == 0
    # b is fed again from behind the pages of its own that nobody had taken meanwhile, not from its first token
    assert fed_again and fed_again[0][0] > 0 and fed_again[0][0] % 4 == 0
    assert {s.request_id: s.token_ids for s in done} == {0: expected(a), 1: expected(b)}


@pytest.mark.parametrize("seed", range(6))
def test_random_workloads_with_shared_prefixes_finish_with_the_same_tokens(seed):
    rng = random.Random(50 + seed)
    sched, cache = make(num_pages=rng.choice([16, 24, 40]), page_size=rng.choice([2, 4, 8]),
                        max_num_seqs=rng.choice([2, 4]), budget=rng.choice([8, 24, 64]), prefix_caching=True)
    stems = [[rng.randrange(900) for _ in range(40)] for _ in range(2)]
    seqs = []
    for i in range(14):
        ids = rng.choice(stems)[:rng.randint(1, 14)] + [rng.randrange(900) for _ in range(rng.randint(0, 6))]
        seqs.append(Sequence(i, ids, len(ids), SamplingParams(max_tokens=rng.randint(1, 12))))
    want = {s.request_id: expected(s) for s in seqs}
    if seed % 2:
        done, _ = run_ahead(sched, cache, seqs)
    else:
        done, _ = run(sched, cache, seqs)
    assert {s.request_id: s.token_ids for s in done} == want
    assert cache.prefix_hit_tokens > 0
    assert not cache.requests and all(g.pool.num_free == g.pool.num_pages for g in cache.groups)


def test_abort_gives_everything_back_wherever_the_request_stands():
    sched, cache = make(num_pages=16, budget=8, max_num_seqs=2)
    seqs = [seq(i, 10, max_tokens=20) for i in range(3)]
    for s in seqs:
        sched.add(s)
    free0 = cache.groups[0].pool.num_free
    batch = sched.schedule()                       # request 0 gets a portion; 1 and 2 wait or start
    sched.postprocess(batch, [fake_token(b.seq.token_ids) for b in batch if b.samples], now=1.0)
    running = {s.request_id for s in sched.running}
    assert 0 in running and 2 not in running
    # a running request in the middle of its prompt, and one that still waits
    a = sched.abort(0, now=2.0)
    w = sched.abort(2, now=2.0)
    assert a is seqs[0] and a.state is State.FINISHED and a.finish_reason == "aborted" and a.finish_ts == 2.0
    assert w is seqs[2] and w.finish_reason == "aborted" and w.num_output_tokens == 0
    assert sched.abort(0) is None and sched.abort(77) is None
    assert not cache.has(0) and not cache.has(2)
    cache.check()
    # the rest runs to its end as if the others had never been there
    done = []
    steps = 0
    while not sched.is_finished():
        batch = sched.schedule()
        assert all(b.seq.request_id == 1 for b in batch)
        done += sched.postprocess(batch, [fake_token(b.seq.token_ids) for b in batch if b.samples], now=3.0)
        steps += 1
        assert steps < 100
    assert [s.request_id for s in done] == [1] and done[0].token_ids == expected(seqs[1])
    assert not cache.requests and cache.groups[0].pool.num_free == free0
    # a step that is on the device when its request is aborted: the token that arrives is passed over
    sched2, cache2 = make(num_pages=16, budget=8)
    b = seq(5, 4, max_tokens=20)
    sched2.add(b)
    batch = sched2.schedule()
    sched2.advance(batch)
    sched2.abort(5)
    assert sched2.absorb(batch, [123]) == [] and b.num_output_tokens == 0 and sched2.is_finished()
    cache2.check()


def test_a_window_smaller_than_its_pool_needs_is_refused_when_the_request_is_added():
    # a window of 40 with pages of 16 holds up to 4 pages token by token: 3 pages could never do
    sched, cache = make(num_pages=3, page_size=16, window=40, max_model_len=512)
    with pytest.raises(ValueError, match="window of 40"):
        sched.add(seq(0, 100, max_tokens=50))
    sched, cache = make(num_pages=4, page_size=16, window=40, max_model_len=512)
    a = seq(0, 100, max_tokens=50)
    done, _ = run(sched, cache, [a])
    assert done[0].token_ids == expected(a)
    # a short request needs no more than its own length
    sched, cache = make(num_pages=2, page_size=16, window=40, max_model_len=512)
    b = seq(1, 20, max_tokens=10)
    done, _ = run(sched, cache, [b])
    assert done[0].token_ids == expected(b)
