"""The scheduler's decisions (CPU), driven against the real cache manager."""
import random

import pytest

from photon_infer_amd import RequestError
from photon_infer_amd.cache import CacheManager
from photon_infer_amd.engine.scheduler import ContinuousBatchScheduler, RequestState
from photon_infer_amd.sampling import SamplingParams


def make(pages=64, page=4, slots=4, budget=16, chunk=8, max_len=128):
    cache = CacheManager([None], page, pages, slots, max_len)
    return cache, ContinuousBatchScheduler(cache, slots, budget, chunk, max_len)


def run_step(cache, sched, batch, eos=(), next_token=lambda r: 1):
    """What the engine does with a scheduled batch, without a model."""
    done = []
    for req, n in batch.items:
        cache.reserve(req.request_id, n)
        cache.commit(req.request_id, n)
        ends = req.num_computed_tokens + n == req.total_tokens()
        req.add_computed_tokens(n)
        if ends and not req.add_token(next_token(req), eos, sched.max_model_len):
            done.append(req)
    sched.update_after_step(done)
    cache.check_invariants()
    return done


def test_prompts_are_cut_under_the_budget_and_decodes_go_first():
    cache, s = make(budget=10, chunk=6)
    a = s.add_request(list(range(13)), SamplingParams(max_new_tokens=3))
    b1 = s.schedule_next_batch()
    assert [(r.request_id, n) for r, n in b1.items] == [(a, 6)]
    run_step(cache, s, b1)
    b = s.add_request(list(range(9)), SamplingParams(max_new_tokens=3))
    b2 = s.schedule_next_batch()                 # a continues (6), b admitted with what is left (4)
    assert [(r.request_id, n) for r, n in b2.items] == [(a, 6), (b, 4)]
    run_step(cache, s, b2)
    b3 = s.schedule_next_batch()                 # a: last prompt token; b: 5 more
    assert [(r.request_id, n) for r, n in b3.items] == [(a, 1), (b, 5)]
    run_step(cache, s, b3)
    ra, rb = s.get_request(a), s.get_request(b)
    assert ra.num_generated() == 1 and ra.is_decode() and rb.num_generated() == 1
    b4 = s.schedule_next_batch()
    assert [(r.request_id, n) for r, n in b4.items] == [(a, 1), (b, 1)]
    assert b4.num_tokens() <= 10


def test_the_last_prompt_token_is_not_fed_twice():
    cache, s = make()
    a = s.add_request([5, 6, 7], SamplingParams(max_new_tokens=2))
    req = s.get_request(a)
    fed = []
    while s.has_work():
        batch = s.schedule_next_batch()
        for r, n in batch.items:
            fed += r.next_tokens(n)
        run_step(cache, s, batch, next_token=lambda r: 40 + r.num_generated())
    assert fed == [5, 6, 7, 40]                   # the second sampled token ends the request unfed
    assert req.generated_tokens == [40, 41] and req.finish_reason == "length"
    assert cache.num_live == 0 and cache.free_pages() == 64


def test_first_come_first_served_and_slots():
    cache, s = make(slots=2, budget=64, chunk=64)
    ids = [s.add_request([1] * 4, SamplingParams(max_new_tokens=2)) for _ in range(5)]
    order = []
    while s.has_work():
        batch = s.schedule_next_batch()
        assert batch.batch_size() <= 2
        for r, _ in batch.items:
            if r.request_id not in order:
                order.append(r.request_id)
        run_step(cache, s, batch)
    assert order == ids
    assert s.get_stats().num_finished == 5


def test_eos_and_max_model_len_end_a_request():
    cache, s = make(max_len=6)
    a = s.add_request([1, 2, 3], SamplingParams(max_new_tokens=50))
    b = s.add_request([1, 2, 3], SamplingParams(max_new_tokens=50))
    while s.has_work():
        run_step(cache, s, s.schedule_next_batch(), eos=(9,),
                 next_token=lambda r: 9 if r.request_id == a and r.num_generated() == 1 else 4)
    ra, rb = s.get_request(a), s.get_request(b)
    assert ra.generated_tokens == [4, 9] and ra.finish_reason == "eos"
    assert rb.finish_reason == "max_model_len" and rb.total_tokens() == 7   # the 7th could not be fed


def test_rejected_requests():
    cache, s = make(max_len=8)
    with pytest.raises(RequestError):
        s.add_request([])
    with pytest.raises(RequestError, match="longer"):
        s.add_request([1] * 9)
    with pytest.raises(RequestError):
        s.add_request([1], SamplingParams(max_new_tokens=0))


def test_out_of_pages_preempts_the_newest_and_recomputes_it():
    # 6 pages of 4 tokens; two requests that each grow to 16 tokens cannot both stay
    cache, s = make(pages=6, budget=32, chunk=32)
    a = s.add_request([1] * 7, SamplingParams(max_new_tokens=9))
    b = s.add_request([2] * 7, SamplingParams(max_new_tokens=9))
    ra, rb = s.get_request(a), s.get_request(b)
    saw_preempt = False
    guard = 0
    while s.has_work():
        guard += 1
        assert guard < 200
        batch = s.schedule_next_batch()
        if batch.preempted:
            saw_preempt = True
            assert batch.preempted == [rb]                 # the newest, never the oldest
            assert rb.state is RequestState.WAITING and rb.num_computed_tokens == 0
            assert s.waiting[0] is rb and rb.request_id not in cache
            kept = list(rb.generated_tokens)
        run_step(cache, s, batch, next_token=lambda r: 10 + r.num_generated())
    assert saw_preempt and s.get_stats().num_preemptions >= 1
    # both finish with the full count and the tokens generated before preemption are kept
    assert ra.generated_tokens == [10 + i for i in range(9)]
    assert rb.generated_tokens == [10 + i for i in range(9)]
    assert rb.generated_tokens[:len(kept)] == kept
    assert cache.free_pages() == 6 and cache.num_live == 0


def test_a_request_waits_until_its_whole_prompt_has_room():
    """Admission wants room for the whole prompt, not only for the first portion: a request
    let in on less would be preempted before its prompt is through."""
    cache, s = make(pages=8, page=4, budget=16, chunk=4)         # 32 tokens in the pool
    a = s.add_request(list(range(20)), SamplingParams(max_new_tokens=4))
    b1 = s.schedule_next_batch()
    run_step(cache, s, b1)                                       # a holds one page, seven are free
    b = s.add_request(list(range(30)), SamplingParams(max_new_tokens=2))      # 8 pages: one portion fits, the prompt does not
    b2 = s.schedule_next_batch()
    assert [(r.request_id, n) for r, n in b2.items] == [(a, 4)]
    assert s.get_request(b).state is RequestState.WAITING
    run_step(cache, s, b2)
    while s.get_request(a).state is not RequestState.FINISHED:   # a runs to its end alone
        batch = s.schedule_next_batch()
        assert all(r.request_id == a for r, _ in batch.items)
        run_step(cache, s, batch)
    b3 = s.schedule_next_batch()                                 # now the pool is empty: b's prompt has room
    assert [(r.request_id, n) for r, n in b3.items] == [(b, 4)]


def test_a_request_that_cannot_fit_alone_is_finished_not_hung():
    cache, s = make(pages=2, budget=64, chunk=64)       # 8 tokens of cache
    a = s.add_request([1] * 12, SamplingParams(max_new_tokens=4))     # can never start
    b = s.add_request([1] * 3, SamplingParams(max_new_tokens=20))     # starts, then outgrows the pool
    guard = 0
    while s.has_work():
        guard += 1
        assert guard < 100
        run_step(cache, s, s.schedule_next_batch())
    ra, rb = s.get_request(a), s.get_request(b)
    assert ra.finish_reason == "out_of_pages" and ra.num_generated() == 0
    assert rb.finish_reason == "out_of_pages" and rb.total_tokens() == 9   # 8 fed + one sampled
    assert cache.free_pages() == 2 and cache.num_live == 0


@pytest.mark.parametrize("seed", range(6))
def test_random_workloads_keep_every_invariant(seed):
    rng = random.Random(seed)
    cache, s = make(pages=rng.choice([10, 16, 40]), slots=rng.choice([2, 4]), budget=rng.choice([5, 12, 40]),
                    chunk=rng.choice([3, 8, 64]), max_len=64)
    ids, computed = [], {}
    pending = [([rng.randrange(50)] * rng.randint(1, 30), rng.randint(1, 12)) for _ in range(12)]
    guard = 0
    while s.has_work() or pending:
        guard += 1
        assert guard < 3000
        while pending and rng.random() < 0.4:
            p, n = pending.pop()
            ids.append(s.add_request(p, SamplingParams(max_new_tokens=n)))
        if not s.has_work():
            continue
        batch = s.schedule_next_batch()
        assert batch.num_tokens() <= s.max_step_tokens and batch.batch_size() <= s.max_batch_size
        assert len({r.request_id for r in batch.requests}) == batch.batch_size()
        for r in batch.preempted:
            computed[r.request_id] = 0
        for r, n in batch.items:
            assert r.state is RequestState.RUNNING and 1 <= n <= s.chunk_size
            assert r.num_computed_tokens >= computed.get(r.request_id, 0)     # monotone but for preemption
            assert cache.length(r.request_id) == r.num_computed_tokens
        run_step(cache, s, batch)
        for r, n in batch.items:
            computed[r.request_id] = r.num_computed_tokens
    for i in ids:
        r = s.get_request(i)
        assert r.is_finished()
        if r.finish_reason == "length":
            assert r.num_generated() == r.max_new_tokens
    assert cache.num_live == 0 and cache.free_pages() == cache.groups[0].pool.num_pages
    cache.check_invariants()


def test_abort_gives_slot_and_pages_back_at_once():
    cache, s = make(pages=16, page=4, slots=2, budget=16, chunk=8)
    a = s.add_request(list(range(10)), SamplingParams(max_new_tokens=50))
    b = s.add_request(list(range(6)), SamplingParams(max_new_tokens=50))
    c = s.add_request(list(range(5)), SamplingParams(max_new_tokens=4))      # waits: two slots only
    for _ in range(3):
        run_step(cache, s, s.schedule_next_batch())
    ra, rb, rc = (s.get_request(i) for i in (a, b, c))
    assert ra.state is RequestState.RUNNING and rb.state is RequestState.RUNNING and rc.state is RequestState.WAITING
    held = cache.free_pages()
    assert s.abort(c)                                        # waiting: leaves the queue, holds nothing
    assert rc.is_finished() and rc.finish_reason == "aborted" and not s.waiting and cache.free_pages() == held
    generated = list(ra.generated_tokens)
    assert s.abort(a)                                        # running: pages and slot are back before the next step
    assert ra.finish_reason == "aborted" and ra.generated_tokens == generated
    assert cache.free_pages() > held and cache.free_slots == 1 and ra not in s.running
    cache.check_invariants()
    assert not s.abort(a) and not s.abort(12345)             # finished, unknown
    d = s.add_request(list(range(7)), SamplingParams(max_new_tokens=3))
    while s.has_work():                                      # the freed slot serves the next request
        run_step(cache, s, s.schedule_next_batch())
    assert s.get_request(d).finish_reason == "length" and rb.finish_reason == "length"
    assert cache.free_pages() == 16 and cache.num_live == 0
    st = s.get_stats()
    assert st.num_aborted == 2 and st.num_finished == 4


@pytest.mark.parametrize("seed", range(5))
def test_random_aborts_lose_no_page(seed):
    rng = random.Random(seed)
    cache, s = make(pages=24, page=4, slots=3, budget=12, chunk=5, max_len=64)
    ids = []
    for step in range(200):
        if rng.random() < 0.3 and len(ids) < 25:
            ids.append(s.add_request([1] * rng.randint(1, 30), SamplingParams(max_new_tokens=rng.randint(1, 12))))
        if ids and rng.random() < 0.15:
            s.abort(rng.choice(ids))
        if s.has_work():
            run_step(cache, s, s.schedule_next_batch())
    for i in ids:
        s.abort(i)
    cache.check_invariants()
    assert cache.free_pages() == 24 and cache.num_live == 0 and not s.has_work()
    assert all(s.get_request(i).is_finished() for i in ids)
