"""The scheduler's decisions (no GPU), with a fake model: the next token is a function of the
tokens so far, so any loss or repetition of work shows in the output."""
import pytest

from deliverance_amd.cache import CacheManager, KVGroupSpec
from deliverance_amd.engine.scheduler import (FINISH_ERROR, FINISH_LENGTH, FINISH_STOP, Scheduler, SchedulerError)
from deliverance_amd.sampling import GeneratorParameters

V = 97


def fake_next(tokens):
    h = 7
    for i, t in enumerate(tokens):
        h = (h * 31 + (i + 1) * (t + 3)) % 1000003
    return h % V


def make(n_pages=64, page=4, max_batch_tokens=16, max_chunk=8, max_num_seqs=4, max_positions=64, eos=(96,)):
    cache = CacheManager([KVGroupSpec((0,), 1, 16, None)], page, [n_pages])
    return Scheduler(cache, max_positions, eos, max_num_seqs, max_batch_tokens, max_chunk), cache


def drive(s, cache, log=None, max_steps=10000):
    """Runs until idle; checks the budget and the cache invariants at every step."""
    seen = {}
    for _ in range(max_steps):
        if not s.has_work():
            break
        batch = s.schedule()
        cache.check()
        if not batch:
            continue
        assert sum(b.n for b in batch) <= s.max_batch_tokens
        assert all(b.n <= s.max_chunk for b in batch)
        assert len({id(b.request) for b in batch}) == len(batch)
        sampled = {}
        for b in batch:
            # the fake model sees exactly the tokens the engine would hold for the request
            assert b.start == b.request.n_computed
            seen[b.request.rid] = seen.get(b.request.rid, 0) + b.n
            if b.samples:
                sampled[b.request.rid] = fake_next(b.request.tokens_from(0, b.start + b.n))
        if log is not None:
            log.append([(b.request.rid, b.start, b.n) for b in batch])
        s.complete(batch, sampled)
        cache.check()
    else:
        raise AssertionError("the scheduler did not come to rest")
    return seen


def expected(prompt, n):
    toks = list(prompt)
    for _ in range(n):
        toks.append(fake_next(toks))
    return toks[len(prompt):]


def test_max_tokens_gives_exactly_that_many():
    # the reference: maxTokens=8 gives exactly 8 generated tokens
    # (core/src/test/java/io/teknek/deliverance/model/MaxTokenTest.java:113-121)
    s, cache = make(eos=())
    r = s.add("a", [1, 2, 3], GeneratorParameters(max_tokens=8))
    drive(s, cache)
    assert r.output == expected([1, 2, 3], 8) and r.finish_reason == FINISH_LENGTH
    assert cache.pools[0].n_free == 64


def test_prompts_are_cut_under_the_budget_decodes_first():
    s, cache = make(max_batch_tokens=10, max_chunk=6, eos=())
    s.add("a", list(range(1, 4)), GeneratorParameters(max_tokens=6))
    s.add("b", list(range(1, 21)), GeneratorParameters(max_tokens=2))
    log = []
    drive(s, cache, log)
    assert log[0] == [("a", 0, 3), ("b", 0, 6)]
    # from now on 'a' decodes (one token, first in the batch) while 'b' goes on with portions
    assert log[1] == [("a", 3, 1), ("b", 6, 6)]
    assert log[2] == [("a", 4, 1), ("b", 12, 6)]
    assert log[3] == [("a", 5, 1), ("b", 18, 2)]
    assert [r.rid for r in s.finished] == ["b", "a"] or {r.rid for r in s.finished} == {"a", "b"}
    for r in s.finished:
        assert r.output == expected(r.prompt, r.params.max_tokens)


def test_end_token_stops_and_ntokens_bounds_positions():
    s, cache = make(eos=(fake_next([5, 6]),))
    r = s.add("a", [5, 6], GeneratorParameters())
    drive(s, cache)
    assert r.finish_reason == FINISH_STOP and len(r.output) == 1      # the end token is counted
    s2, cache2 = make(eos=())
    r2 = s2.add("b", [1, 2, 3, 4], GeneratorParameters(ntokens=10))
    drive(s2, cache2)
    # positions 0..9 are computed; the token sampled after position 9 is the last
    assert r2.finish_reason == FINISH_LENGTH and len(r2.prompt) + len(r2.output) == 11
    s3, cache3 = make(eos=(fake_next([5, 6]),))
    r3 = s3.add("c", [5, 6], GeneratorParameters(ignore_eos=True, max_tokens=3))
    drive(s3, cache3)
    assert len(r3.output) == 3


def test_admission_rules():
    s, _ = make(max_positions=16)
    with pytest.raises(SchedulerError, match="Prompt exceeds ntokens"):
        s.add("a", list(range(16)), GeneratorParameters())
    with pytest.raises(SchedulerError, match="exceed config length"):
        s.add("a", [1], GeneratorParameters(ntokens=17))
    with pytest.raises(SchedulerError, match="Prompt exceeds ntokens"):
        s.add("a", [1, 2, 3], GeneratorParameters(ntokens=3))
    with pytest.raises(SchedulerError):
        s.add("a", [], GeneratorParameters())
    s.add("a", [1], GeneratorParameters())
    with pytest.raises(SchedulerError, match="already queued"):
        s.add("a", [1], GeneratorParameters())
    with pytest.raises(ValueError):
        s.add("b", [1], GeneratorParameters(top_p=1.5))


def test_no_more_live_requests_than_allowed_and_everyone_finishes():
    s, cache = make(max_num_seqs=2, eos=())
    reqs = [s.add(i, [i + 1] * (3 + i), GeneratorParameters(max_tokens=4 + i)) for i in range(6)]
    for _ in range(1000):
        if not s.has_work():
            break
        batch = s.schedule()
        assert len(s.running) <= 2
        s.complete(batch, {b.request.rid: fake_next(b.request.tokens_from(0, b.start + b.n)) for b in batch if b.samples})
    assert all(r.output == expected(r.prompt, r.params.max_tokens) for r in reqs)
    assert cache.pools[0].n_free == 64


def test_when_pages_run_out_the_newest_request_is_computed_again():
    # 6 pages of 4 rows; two requests that together outgrow the pool
    s, cache = make(n_pages=6, max_batch_tokens=32, max_chunk=32, eos=())
    a = s.add("a", [1, 2, 3, 4, 5], GeneratorParameters(max_tokens=14))
    b = s.add("b", [9, 8, 7], GeneratorParameters(max_tokens=14))
    log = []
    drive(s, cache, log)
    assert s.counters["preemptions"] >= 1 and b.n_preempted >= 1 and a.n_preempted == 0
    # the preempted request ends with the tokens it would have had without preemption
    assert a.output == expected(a.prompt, 14) and b.output == expected(b.prompt, 14)
    # after coming back it is computed again from its first token
    restarts = [step for step in log for (rid, start, n) in step if rid == "b" and start == 0]
    assert len(restarts) >= 2
    assert cache.pools[0].n_free == 6


def test_a_request_that_cannot_fit_alone_fails_cleanly():
    s, cache = make(n_pages=2, eos=())
    r = s.add("a", [1, 2, 3], GeneratorParameters(max_tokens=20))
    drive(s, cache)
    assert r.finish_reason == FINISH_ERROR and "more cache than the whole pool" in r.error
    assert len(r.output) >= 5 and r.output == expected(r.prompt, len(r.output))
    assert cache.pools[0].n_free == 2 and not s.has_work()


def test_cancel_returns_what_the_request_holds():
    s, cache = make(eos=())
    s.add("a", [1, 2, 3], GeneratorParameters(max_tokens=50))
    s.add("b", [4, 5], GeneratorParameters(max_tokens=50))
    batch = s.schedule()
    s.complete(batch, {b.request.rid: 1 for b in batch if b.samples})
    assert s.cancel("a") and not s.cancel("zzz")
    cache.check()
    assert [r.rid for r in s.running] == ["b"]
    s.cancel("b")
    assert cache.pools[0].n_free == 64 and not s.has_work()


@pytest.mark.parametrize("seed", range(4))
def test_random_loads_with_small_pools(seed):
    import random
    rng = random.Random(seed)
    s, cache = make(n_pages=rng.randint(8, 14), page=4, max_batch_tokens=rng.choice([6, 12, 32]),
                    max_chunk=rng.choice([2, 5, 32]), max_num_seqs=rng.randint(1, 4), eos=())
    reqs = []
    for i in range(10):
        prompt = [rng.randrange(V) for _ in range(rng.randint(1, 12))]
        reqs.append(s.add(i, prompt, GeneratorParameters(max_tokens=rng.randint(1, 12))))
    drive(s, cache)
    for r in reqs:
        assert r.finish_reason == FINISH_LENGTH
        assert r.output == expected(r.prompt, r.params.max_tokens)
    assert cache.pools[0].n_free == cache.pools[0].n_pages


def drive_ahead(s, cache, max_steps=10000):
    """As ``drive``, but each step is decided ahead of the one before where the scheduler allows
    it: the fake model then only learns a request's token when the older step is completed, and a
    request that ended meanwhile has one step too many, whose result is dropped.  Returns how many
    steps were decided ahead."""
    inflight = None          # (batch, sampled tokens by request id), launched but not completed
    n_ahead = 0
    reached = {}             # request -> (positions launched so far, preemptions seen): no gap, no repeat

    def launch(batch, prev):
        sampled = {}
        for b in batch:
            at, pre = reached.get(b.request.rid, (0, b.request.n_preempted))
            if pre != b.request.n_preempted:
                at = 0                                         # preempted: computed again from the start
            assert b.start == at, f"{b.request.rid}: portion starts at {b.start}, {at} positions were launched"
            reached[b.request.rid] = (b.start + b.n, b.request.n_preempted)
            if b.samples:
                toks = b.request.tokens_from(0, min(b.start + b.n, b.request.n_tokens))
                if b.start + b.n > b.request.n_tokens:         # its last token is the one the older step sampled
                    toks.append(prev[b.request.rid])
                sampled[b.request.rid] = fake_next(toks)
        return batch, sampled

    for _ in range(max_steps):
        if inflight is not None:
            nxt = s.schedule_ahead(inflight[0])
            cache.check()
            launched = None
            if nxt is not None:
                n_ahead += 1
                for b in nxt:        # only the token that is still being sampled may be unknown
                    if b.start + b.n > b.request.n_tokens:
                        assert b.n == 1 and b.samples and b.start == b.request.n_tokens
                        assert b.request.rid in inflight[1]
                assert sum(b.n for b in nxt) <= s.max_batch_tokens and all(b.n <= s.max_chunk for b in nxt)
                assert len({id(b.request) for b in nxt}) == len(nxt)
                launched = launch(nxt, inflight[1])
            s.complete(inflight[0], {rid: t for rid, t in inflight[1].items()})
            cache.check()
            inflight = launched
            if inflight is not None:
                continue
        if not s.has_work():
            break
        batch = s.schedule()
        cache.check()
        if batch:
            assert all(b.start == b.request.n_computed for b in batch)
            inflight = launch(batch, None)
    else:
        raise AssertionError("the scheduler did not come to rest")
    return n_ahead


def test_steps_decided_ahead_give_the_same_tokens():
    s, cache = make(max_num_seqs=3)
    a = s.add("a", [1, 2, 3], GeneratorParameters(max_tokens=9))
    b = s.add("b", [4, 5, 6, 7, 8], GeneratorParameters(max_tokens=4))
    free = expected([9, 10], 30)
    s.eos = {free[6]}
    c = s.add("c", [9, 10], GeneratorParameters(max_tokens=30))
    n_ahead = drive_ahead(s, cache)
    assert n_ahead >= 8
    assert a.output == expected(a.prompt, 9) and a.finish_reason == FINISH_LENGTH
    assert b.output == expected(b.prompt, 4) and b.finish_reason == FINISH_LENGTH
    assert c.output == free[:free.index(free[6]) + 1] and c.finish_reason == FINISH_STOP
    assert cache.pools[0].n_free == cache.pools[0].n_pages and cache.live() == []


def test_what_is_decided_ahead_and_what_waits_for_the_tokens():
    s, cache = make(n_pages=3, page=4, max_num_seqs=2)
    a = s.add("a", [1, 2, 3], GeneratorParameters(max_tokens=20, ignore_eos=True))
    batch = s.schedule()
    assert [(x.request.rid, x.start, x.n, x.samples) for x in batch] == [("a", 0, 3, True)]
    # b arrives while a's prompt runs: a decodes the token that is still being sampled, b is admitted
    b = s.add("b", [4, 5], GeneratorParameters(max_tokens=20, ignore_eos=True))
    ahead = s.schedule_ahead(batch)
    assert [(x.request.rid, x.start, x.n, x.samples) for x in ahead] == [("a", 3, 1, True), ("b", 0, 2, True)]
    assert cache.length("a") == 0 and cache.pending("a") == 4        # both steps' positions are reserved
    s.complete(batch, {"a": 5})
    assert cache.length("a") == 3 and cache.pending("a") == 1
    batch, ahead = ahead, s.schedule_ahead(ahead)
    assert [(x.request.rid, x.start, x.n) for x in ahead] == [("a", 4, 1), ("b", 2, 1)]
    assert cache.pools[0].n_free == 0                                # a holds 2 pages (5 positions), b 1 (3 positions)
    s.complete(batch, {"a": 6, "b": 7})
    batch, ahead = ahead, s.schedule_ahead(ahead)                    # a at 5, b at 3: both still fit their pages
    assert [(x.request.rid, x.start, x.n) for x in ahead] == [("a", 5, 1), ("b", 3, 1)]
    s.complete(batch, {"a": 8, "b": 9})
    # b's position 4 needs a page that is not there: who gives way is decided with the tokens known
    assert s.schedule_ahead(ahead) is None
    assert cache.length("a") == 5 and cache.pending("a") == 1 and cache.length("b") == 3 and cache.pending("b") == 1
    cache.check()
    s.complete(ahead, {"a": 10, "b": 11})
    batch = s.schedule()
    # b gave its page back and starts again from its tokens, as far as the one free page reaches
    assert [(x.request.rid, x.start, x.n) for x in batch] == [("a", 6, 1), ("b", 0, 4)] and b.n_preempted == 1
    # a prompt in portions goes on ahead as well: nothing of it depends on a token
    s2, cache2 = make(max_chunk=4, max_batch_tokens=6)
    c = s2.add("c", list(range(10)), GeneratorParameters(max_tokens=3, ignore_eos=True))
    first = s2.schedule()
    second = s2.schedule_ahead(first)
    third = s2.schedule_ahead(second)
    fourth = s2.schedule_ahead(third)
    assert [[(x.start, x.n, x.samples) for x in st] for st in (first, second, third, fourth)] == \
        [[(0, 4, False)], [(4, 4, False)], [(8, 2, True)], [(10, 1, True)]]


@pytest.mark.parametrize("seed", range(4))
def test_random_loads_decided_ahead(seed):
    import random
    rng = random.Random(100 + seed)
    s, cache = make(n_pages=rng.randint(8, 14), page=4, max_batch_tokens=rng.choice([6, 12, 32]),
                    max_chunk=rng.choice([2, 5, 32]), max_num_seqs=rng.randint(1, 4), eos=(5, 6, 7, 8, 9, 10))
    reqs = []
    for i in range(10):
        prompt = [rng.randrange(V) for _ in range(rng.randint(1, 12))]
        reqs.append(s.add(i, prompt, GeneratorParameters(max_tokens=rng.randint(1, 12))))
    drive_ahead(s, cache)
    for r in reqs:
        want = expected(r.prompt, r.params.max_tokens)
        stop = next((i for i, t in enumerate(want) if t in s.eos), None)
        if stop is not None and stop + 1 < len(want):
            assert r.finish_reason == FINISH_STOP and r.output == want[:stop + 1]
        else:
            assert r.output == want
    assert cache.pools[0].n_free == cache.pools[0].n_pages
