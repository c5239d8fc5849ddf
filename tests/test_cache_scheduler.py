"""The library's cache manager (no page lost, held twice or freed twice, under random orders
of requests; windows; state slots) and its scheduler's decisions, by themselves, without a GPU
(the objects live in the library; the tests drive them through its host-object calls)."""
import random

import pytest

from celeg_amd.cache import CacheManager, PageError, PagePool, cache_layout
from celeg_amd.engine import RequestOptions, RequestStatus, Scheduler, SchedulerOptions
from celeg_amd.sampling import GREEDY, GenerationConfig


# ---------------------------------------------------------------- page pool
def test_pool_behaviour_of_the_reference():
    # tests/concurrent_policy_test.cpp:8-50
    pool = PagePool(8, 16)
    assert pool.allocate_tokens(0) == []
    assert pool.allocate_tokens(1) == [0]
    three = pool.allocate_tokens(33)
    assert three == [1, 2, 3]
    assert pool.allocate_tokens(80) is None and pool.n_free == 4      # all or nothing
    pool.retain(three)
    pool.release(three)
    assert pool.n_free == 4
    pool.release(three)
    assert pool.n_free == 7
    with pytest.raises(PageError, match="double"):
        pool.release(three)
    with pytest.raises(PageError):
        pool.release([0, 0])                  # transactional: page 0 is held once
    assert pool.holders(0) == 1
    with pytest.raises(PageError):
        pool.retain([0, 99])
    assert pool.holders(0) == 1
    pool.check()


def make_manager(n_pages=12, slots=4, window=None, max_context=256, extra_group=False):
    groups = [(2, 16, None, 2)]
    uses = {1: (0, 0, True), 3: (0, 1, True)}
    if window or extra_group:
        groups.append((1, 16, window, 1))
        uses[4] = (1, 0, True)
    states = [(0, "bx", (3, 8)), (2, "bx", (3, 8)), (2, "count", (1,), "int32")]
    m = CacheManager(cache_layout(groups, uses, states), page_tokens=16, n_pages=n_pages, max_requests=slots,
                     max_context=max_context)
    m.pool_pages = n_pages if isinstance(n_pages, int) else n_pages[0]
    return m


def test_manager_allocates_covers_and_gives_back():
    m = make_manager()
    s = m.open()
    assert m.prepare(s, 0, 17) and m.pages_held(s) == [[0, 1]]
    assert m.covers(s, 0, 17) and m.covers(s, 17, 15) and not m.covers(s, 17, 16)
    assert m.prepare(s, 17, 1) and m.pages_held(s) == [[0, 1]]        # same page
    assert m.prepare(s, 18, 30) and len(m.pages_held(s)[0]) == 3
    updates = m.drain_table_updates()
    assert updates == [[(s, 0, 0), (s, 1, 1), (s, 2, 2)]] and m.drain_table_updates() == [[]]
    s2 = m.open()
    assert not m.prepare(s2, 0, 16 * 10)                               # 9 free: nothing taken
    assert m.free_pages() == [9] and m.pages_held(s2) == [[]]
    with pytest.raises(ValueError, match="context limit"):
        m.prepare(s2, 250, 10)
    m.close(s)
    assert m.free_pages() == [12]
    with pytest.raises(PageError):
        m.close(s)
    s3 = m.open()
    assert s3 == s                                                     # the slot is used again
    assert m.prepare(s3, 0, 16) and m.pages_held(s3)[0][0] in (0, 1, 2)    # and so are its pages
    m.check()


def test_state_slots_have_regions_of_their_own():
    """Every (run-order entry, state) has a region of a slot's row of bytes: typed, aligned to
    16 bytes, not overlapping; one row per request and one for the null slot.  (That a slot is
    zeroed when a request takes it is checked on the GPU, with a mixer that keeps state.)"""
    m = make_manager()
    st = m.state()
    regions = st["state_regions"]
    assert set(regions) == {"0:bx", "2:bx", "2:count"}
    assert regions["0:bx"]["shape"] == [5, 3, 8] and regions["2:count"]["shape"] == [5, 1]
    assert regions["2:count"]["dtype"] == "int32" and regions["0:bx"]["dtype"] == "float32"
    spans = sorted((r["offset"], r["offset"] + 4 * r["shape"][1] * (r["shape"][2] if len(r["shape"]) > 2 else 1))
                   for r in regions.values())
    assert all(a[1] <= b[0] for a, b in zip(spans, spans[1:]))           # regions do not overlap
    assert all(off % 16 == 0 for off, _ in spans)
    assert st["slot_bytes"] == 96 + 96 + 16 and regions["0:bx"]["slot_stride"] == st["slot_bytes"] // 4
    assert st["null_slot"] == 4 and st["max_pages_per_request"] == 16 and st["n_groups"] == 1


def test_window_group_gives_pages_back_as_the_window_passes():
    m = make_manager(n_pages=6, window=20)
    s = m.open()
    pos = 0
    held = []
    for n in [30, 1, 1, 40, 1, 16, 1, 1]:
        assert m.prepare(s, pos, n)
        assert m.covers(s, pos, n)
        pos += n
        full, win = m.pages_held(s)
        held.append((len(full), len(win)))
        # the window group never holds more than the window plus the step needs
        assert len(win) <= (20 + n + 15) // 16 + 1
        m.check()
    assert held[-1][0] == (pos + 15) // 16 and held[-1][1] <= 3
    assert m.table(1, s, 0) == -1 and m.table(0, s, 0) >= 0
    m.close(s)
    assert m.free_pages() == [6, 6]


def test_groups_allocate_all_or_nothing():
    m = make_manager(n_pages=[8, 2], extra_group=True)
    s = m.open()
    assert not m.prepare(s, 0, 48)        # group 1 has 2 pages, 3 are needed
    assert m.free_pages() == [8, 2]
    assert m.prepare(s, 0, 32) and m.free_pages() == [6, 0]


@pytest.mark.parametrize("seed", range(6))
def test_random_orders_of_requests_lose_nothing(seed):
    rng = random.Random(seed)
    m = make_manager(n_pages=10, slots=3, window=24 if seed % 2 else None, max_context=200)
    live = {}
    for _ in range(400):
        action = rng.random()
        if action < 0.25 and m.n_free_slots:
            live[m.open()] = 0
        elif action < 0.85 and live:
            s = rng.choice(list(live))
            n = rng.choice([1, 1, 1, 2, 7, 16, 33])
            if live[s] + n <= 200 and m.prepare(s, live[s], n):
                assert m.covers(s, live[s], n)
                live[s] += n
        elif live:
            s = rng.choice(list(live))
            m.close(s)
            del live[s]
        m.check()
        for s, n in live.items():     # the full group holds exactly the pages its tokens need
            assert len(m.pages_held(s)[0]) == (n + 15) // 16
    for s in list(live):
        m.close(s)
    assert all(f == 10 for f in m.free_pages()) and m.n_free_slots == 3


# ---------------------------------------------------------------- scheduler
VOCAB = 50


class FakeStep:
    """Stands in for the model: the next token of a request is a function of all the
    tokens it has been fed, so the outcome shows whether every token was fed once, in
    order, at the right position, whatever the schedule."""

    def __init__(self):
        self.fed = {}
        self.batches = []

    def run(self, plan):
        self.batches.append([(e["id"], e["start"], e["count"]) for e in plan])
        out = []
        for e in plan:
            history = self.fed.setdefault(e["slot"], [])
            assert e["start"] <= len(history), "a position was skipped"
            del history[e["start"]:]
            assert len(e["tokens"]) == e["count"]
            history.extend(e["tokens"])
            if e["samples"]:
                out.append(expected_next(history))
        return out


def expected_next(history):
    return (sum((i + 1) * t for i, t in enumerate(history)) * 7 + len(history)) % VOCAB


def expected_output(prompt, n, eos=()):
    seq, out = list(prompt), []
    for _ in range(n):
        t = expected_next(seq)
        seq.append(t); out.append(t)
        if t in eos:
            break
    return out


def make_scheduler(n_pages=64, slots=4, **opts):
    m = make_manager(n_pages=n_pages, slots=slots, max_context=256)
    return Scheduler(m, SchedulerOptions(max_active_requests=slots, **opts), max_context=256,
                     default_eos=()), m


def drive(sched, fake, max_steps=2000):
    steps = 0
    while sched.has_work():
        plan = sched.plan()
        for slot in sched.slot_events()["released"]:
            fake.fed.pop(slot, None)
        if plan:
            sched.accept(fake.run(plan))
        for slot in sched.slot_events()["released"]:
            fake.fed.pop(slot, None)
        steps += 1
        assert steps < max_steps, "the scheduler does not terminate"
        sched.cache.check()
    return steps


def opts(n, **kw):
    return RequestOptions(max_new_tokens=n, generation=GREEDY, **kw)


def test_submission_checks():
    sched, _ = make_scheduler()
    with pytest.raises(ValueError, match="request prompt is empty"):
        sched.submit([], opts(4))
    with pytest.raises(ValueError, match="request prompt exceeds max_context"):
        sched.submit([1] * 300, opts(4))
    with pytest.raises(ValueError, match="max_new_tokens must be positive"):
        sched.submit([1], opts(0))
    with pytest.raises(ValueError, match="prompt plus max_new_tokens exceeds max_context"):
        sched.submit([1] * 250, opts(10))
    with pytest.raises(ValueError, match="top_k"):
        sched.submit([1], RequestOptions(generation=GenerationConfig(top_k=500)))


def test_budget_portions_and_decode_first():
    sched, _ = make_scheduler(max_batched_tokens=32, prefill_chunk_tokens=20)
    fake = FakeStep()
    a = sched.submit(list(range(1, 46)), opts(5))          # 45 tokens
    b = sched.submit(list(range(3, 12)), opts(5))          # 9 tokens
    drive(sched, fake)
    first = fake.batches[0]
    assert first == [(a, 0, 20), (b, 0, 9)]                # portion <= chunk, both in one step
    second = fake.batches[1]
    assert second[0] == (b, 9, 1) and second[1] == (a, 20, 20)   # decode token first, then portion
    assert all(sum(c for _, _, c in batch) <= 32 for batch in fake.batches)
    for rid, prompt in ((a, list(range(1, 46))), (b, list(range(3, 12)))):
        assert sched.request(rid)["generated"] == expected_output(prompt, 5)
        assert sched.request(rid)["status"] == "finished"
    assert sched.cache.n_free_slots == 4 and sched.cache.free_pages() == [64]


def test_priority_then_age_and_end_tokens_and_poll():
    sched, _ = make_scheduler(slots=1)
    fake = FakeStep()
    low = sched.submit([1, 2, 3], opts(3))
    high = sched.submit([4, 5, 6], opts(3, priority=5))
    later = sched.submit([7, 8], opts(3))
    plan = sched.plan()
    assert [e["id"] for e in plan] == [high]
    sched.accept(fake.run(plan))
    status, tokens, _ = sched.poll(high)
    assert status == RequestStatus.DECODING and tokens == expected_output([4, 5, 6], 1)
    assert sched.poll(high)[1] == []                        # drained
    drive(sched, fake)
    order = [batch[0][0] for batch in fake.batches]
    assert order.index(low) < order.index(later)
    # an end token finishes the request and is emitted
    sched2, _ = make_scheduler()
    prompt = [9, 9, 9]
    eos_tok = expected_output(prompt, 3)[1]
    rid = sched2.submit(prompt, opts(10, eos_token_ids=[eos_tok]))
    drive(sched2, FakeStep())
    assert sched2.request(rid)["generated"] == expected_output(prompt, 10, eos=[eos_tok])
    assert sched2.request(rid)["generated"][-1] == eos_tok


def test_portions_cut_by_the_budget_keep_to_the_granule():
    """A portion that the budget cuts short is a multiple of the granule or waits for the next
    step, so that steps repeat few shapes; the prompt's end and the portion size cut as ever,
    and a step is never left empty for it."""
    sched, _ = make_scheduler(n_pages=64, slots=4, prefill_chunk_tokens=64, max_batched_tokens=100,
                              portion_granule=16)
    fake = FakeStep()
    a = sched.submit([1] * 70, opts(3))
    b = sched.submit([2] * 90, opts(3))
    plan = sched.plan()
    assert [(e["id"], e["count"]) for e in plan] == [(a, 64), (b, 32)]     # 36 left: cut to 32
    sched.accept(fake.run(plan))
    plan = sched.plan()
    assert [(e["id"], e["count"]) for e in plan] == [(a, 6), (b, 58)]      # the ends of both prompts
    sched.accept(fake.run(plan))
    drive(sched, fake)
    assert sched.request(a)["generated"] == expected_output([1] * 70, 3)
    assert sched.request(b)["generated"] == expected_output([2] * 90, 3)
    # a budget below the granule: the first portion of a step is cut at the budget all the same
    sched2, _ = make_scheduler(prefill_chunk_tokens=64, max_batched_tokens=10, portion_granule=16)
    c = sched2.submit([3] * 25, opts(2))
    plan = sched2.plan()
    assert [(e["id"], e["count"]) for e in plan] == [(c, 10)]
    sched2.accept(fake.run(plan))
    drive(sched2, fake)
    assert sched2.request(c)["generated"] == expected_output([3] * 25, 2)


def test_admission_waits_for_pages_and_slots():
    sched, m = make_scheduler(n_pages=4, slots=2, prefill_chunk_tokens=64, max_batched_tokens=64)
    fake = FakeStep()
    a = sched.submit([1] * 40, opts(4))        # 3 pages
    b = sched.submit([2] * 40, opts(4))        # 3 pages: does not fit beside a
    plan = sched.plan()
    assert [(e["id"], e["count"]) for e in plan] == [(a, 40), (b, 16)]   # cut to the free page
    sched.accept(fake.run(plan))
    drive(sched, fake)
    assert sched.request(a)["generated"] == expected_output([1] * 40, 4)
    assert sched.request(b)["generated"] == expected_output([2] * 40, 4)


def test_out_of_pages_stalls_then_preempts_the_youngest_and_still_gives_the_same_tokens():
    sched, m = make_scheduler(n_pages=6, slots=3, prefill_chunk_tokens=64, max_batched_tokens=128)
    fake = FakeStep()
    prompts = [[1 + i] * 30 for i in range(3)]               # 2 pages each: the pool is full
    ids = [sched.submit(p, opts(40)) for p in prompts]       # each grows to 70 tokens = 5 pages
    drive(sched, fake)
    assert sched.stats["preemptions"] > 0 and sched.stats["stalled_decodes"] > 0
    for rid, p in zip(ids, prompts):
        assert sched.request(rid)["status"] == "finished"
        assert sched.request(rid)["generated"] == expected_output(p, 40)
    assert sched.request(ids[0])["preemptions"] == 0           # the oldest is never the victim
    assert m.free_pages() == [6] and m.n_free_slots == 3


def test_request_that_can_never_fit_fails_and_others_go_on():
    sched, m = make_scheduler(n_pages=3, slots=2, prefill_chunk_tokens=256, max_batched_tokens=256)
    fake = FakeStep()
    big = sched.submit([1] * 100, opts(4))                   # 7 pages > 3
    small = sched.submit([2] * 10, opts(4))
    drive(sched, fake)
    assert sched.request(big)["status"] == "failed"
    assert "more cache pages" in sched.request(big)["error"]
    assert sched.request(small)["generated"] == expected_output([2] * 10, 4)


def test_guaranteed_policy_reserves_up_front():
    sched, m = make_scheduler(n_pages=6, slots=3, policy="guaranteed_no_evict",
                              prefill_chunk_tokens=64, max_batched_tokens=128)
    fake = FakeStep()
    ids = [sched.submit([1 + i] * 30, opts(40)) for i in range(3)]    # 5 pages each
    plan = sched.plan()
    assert [e["id"] for e in plan] == [ids[0]] and m.free_pages() == [1]
    sched.accept(fake.run(plan))
    drive(sched, fake)
    assert sched.stats["preemptions"] == 0 and sched.stats["stalled_decodes"] == 0
    assert all(sched.request(r)["generated"] == expected_output([1 + i] * 30, 40)
               for i, r in enumerate(ids))


def test_cancel_frees_everything():
    sched, m = make_scheduler()
    fake = FakeStep()
    a = sched.submit([1] * 20, opts(50))
    b = sched.submit([2] * 20, opts(5))
    for _ in range(3):
        plan = sched.plan(); sched.accept(fake.run(plan))
    sched.cancel(a)
    drive(sched, fake)
    assert sched.request(a)["status"] == "cancelled"
    assert 0 < len(sched.request(a)["generated"]) < 50
    assert sched.request(b)["generated"] == expected_output([2] * 20, 5)
    assert m.free_pages() == [64] and m.n_free_slots == 4


def test_release_forgets_an_ended_request_and_no_other():
    """The record of a request stays until it is released (the reference's release,
    src/backend/cuda/runtime/request_lifecycle.cpp:47-55): refused while the request is queued or
    running, and the others go on as if nothing had happened."""
    sched, m = make_scheduler()
    fake = FakeStep()
    a = sched.submit([1] * 20, opts(3))
    b = sched.submit([2] * 20, opts(30))
    assert sched.release(a) is False                 # queued
    plan = sched.plan(); sched.accept(fake.run(plan))
    assert sched.release(a) is False                 # running
    while sched.request(a)["status"] != "finished":
        plan = sched.plan(); sched.accept(fake.run(plan))
    assert sched.poll(a)[1] == expected_output([1] * 20, 3)
    assert sched.release(a) is True
    with pytest.raises(ValueError, match="unknown request id"):
        sched.request(a)
    with pytest.raises(ValueError, match="unknown request id"):
        sched.release(a)
    c = sched.submit([3] * 10, opts(4))              # ids are not given out again
    assert c not in (a, b)
    drive(sched, fake)
    assert sched.request(b)["generated"] == expected_output([2] * 20, 30)
    assert sched.request(c)["generated"] == expected_output([3] * 10, 4)
    assert sched.release(b) and sched.release(c)
    assert m.free_pages() == [64] and m.n_free_slots == 4


@pytest.mark.parametrize("seed", range(4))
def test_random_workloads_terminate_with_the_right_tokens(seed):
    rng = random.Random(seed)
    sched, m = make_scheduler(n_pages=rng.choice([8, 12, 20]), slots=rng.choice([2, 3, 4]),
                              prefill_chunk_tokens=rng.choice([8, 32]),
                              max_batched_tokens=rng.choice([16, 48]))
    fake = FakeStep()
    work = []
    for _ in range(10):
        prompt = [rng.randrange(VOCAB) for _ in range(rng.choice([1, 5, 17, 40, 64]))]
        n = rng.choice([1, 8, 30])
        work.append((sched.submit(prompt, opts(n)), prompt, n))
    drive(sched, fake)
    for rid, prompt, n in work:
        assert sched.request(rid)["generated"] == expected_output(prompt, n)
    assert m.free_pages() == [m.pool_pages] and m.n_free_slots == m.max_requests


def test_a_failed_step_fails_its_requests_and_frees_what_they_hold():
    """What the engine does when launching or completing a step throws: the step's requests
    become Failed with the message, their pages and slots go back, and the others go on
    (src/backend/cuda/runtime/request_lifecycle.cpp:200-218)."""
    sched, m = make_scheduler(n_pages=16, slots=3, prefill_chunk_tokens=64, max_batched_tokens=64)
    fake = FakeStep()
    a = sched.submit([1] * 20, opts(5))
    b = sched.submit([2] * 20, opts(5))
    plan = sched.plan()
    assert {e["id"] for e in plan} == {a, b}
    sched.fail("HIP error 700 in a kernel")
    for rid in (a, b):
        status, tokens, error = sched.poll(rid)
        assert status == RequestStatus.FAILED and tokens == [] and "HIP error 700" in error
    assert m.free_pages() == [16] and m.n_free_slots == 3 and not sched.has_work()
    assert sorted(sched.slot_events()["released"]) == [0, 1]
    c = sched.submit([3] * 10, opts(4))
    drive(sched, fake)
    assert sched.request(c)["generated"] == expected_output([3] * 10, 4)
    m.check()


def test_latencies_are_recorded_per_request():
    sched, _ = make_scheduler()
    fake = FakeStep()
    rid = sched.submit([1, 2, 3], opts(4))
    drive(sched, fake)
    r = sched.request(rid)
    assert r["ttft_seconds"] >= 0 and r["itl_count"] == 3
