"""The scheduler's decisions, on the CPU, with a made-up token source instead of a model."""
import pytest

from kv_cache_optimization_for_llm_amd.cache.manager import CacheManager
from kv_cache_optimization_for_llm_amd.engine.scheduler import (Request, Scheduler, reservation_tokens)
from kv_cache_optimization_for_llm_amd.parts.base import attention_cache_spec

SPEC = attention_cache_spec(2, 16)
EOS = 7


def cache(pages=64, seqs=8, mode="paged", page=16, max_len=512):
    return CacheManager([(SPEC, [0, 1])], {}, page_size=page, num_pages=pages, max_seqs=seqs,
                        max_seq_len=max_len, mode=mode)


def fake_token(request_id, position):
    """What 'the model' samples for the token that will sit at ``position``: a pure function, as
    greedy decoding of a fixed model is."""
    t = (request_id * 31 + position * 17) % 97 + 8
    return t


def run(s, max_steps=10000, on_plan=None):
    """Runs to idle; returns ({(id, seq): tokens}, {(id, seq): reason}, all events, plans)."""
    out, reasons, events, plans = {}, {}, [], []
    for _ in range(max_steps):
        if s.idle():
            break
        plan = s.plan()
        s.cache.check()
        plans.append(plan)
        if on_plan:
            on_plan(plan)
        evs = list(plan.events)
        for e in plan.entries:
            assert s.cache.grow(e.seq.seat, e.start + len(e.tokens)), "the plan promised pages it cannot get"
        sampled = [fake_token(e.seq.request.id, e.start + len(e.tokens)) for e in plan.entries if e.sample]
        evs += s.complete(plan, sampled)
        s.cache.check()
        for ev in evs:
            key = (ev.request_id, ev.seq_index)
            if ev.kind == "token":
                out.setdefault(key, []).append(ev.token)
            elif ev.kind in ("done", "rejected"):
                reasons[key] = ev.reason
        events += evs
    assert s.idle(), "the scheduler did not finish"
    return out, reasons, events, plans


def test_budget_goes_to_decodes_first_then_to_prompt_portions_in_order():
    s = Scheduler(cache(), max_batch_tokens=40, chunk_size=24, ignore_eos=True)
    s.add(Request(0, list(range(8, 38)), 5))          # 30 tokens
    s.add(Request(1, list(range(8, 58)), 5))          # 50 tokens
    p = s.plan()
    assert [(e.seq.request.id, len(e.tokens), e.sample) for e in p.entries] == [(0, 24, False), (1, 16, False)]
    s.complete(p, [])
    p = s.plan()                                       # 0 finishes its prompt, 1 goes on
    assert [(e.seq.request.id, e.start, len(e.tokens), e.sample) for e in p.entries] == \
        [(0, 24, 6, True), (1, 16, 24, False)]
    s.complete(p, [fake_token(0, 30)])
    p = s.plan()                                       # 0 decodes first, then 1's last portion
    assert [(e.seq.request.id, len(e.tokens), e.sample) for e in p.entries] == [(0, 1, True), (1, 10, True)]
    assert p.entries[0].tokens == [fake_token(0, 30)] and p.num_tokens <= 40


def test_every_request_emits_exactly_its_budget_and_order_is_fcfs():
    s = Scheduler(cache(), max_batch_tokens=64, chunk_size=16, ignore_eos=True)
    lens = [5, 17, 33, 70, 1, 9]
    for i, n in enumerate(lens):
        s.add(Request(i, [8 + (j % 50) for j in range(n)], 8 + i))
    out, reasons, events, plans = run(s)
    for i, n in enumerate(lens):
        assert out[(i, 0)] == [fake_token(i, n + k) for k in range(8 + i)]
        assert reasons[(i, 0)] == "length"
    first_seen = []
    for p in plans:
        for e in p.entries:
            if e.seq.request.id not in first_seen:
                first_seen.append(e.seq.request.id)
    assert first_seen == sorted(first_seen)
    assert all(p.num_tokens <= 64 for p in plans)
    assert s.cache.free_seats == 8 and s.cache.groups[0].free_pages() == 64


def test_eos_ends_a_request_and_is_not_emitted():
    s = Scheduler(cache(), eos_token_ids=[fake_token(3, 12)], max_batch_tokens=64)
    s.add(Request(3, list(range(10, 20)), 20))
    out, reasons, events, _ = run(s)
    assert out[(3, 0)] == [fake_token(3, 10), fake_token(3, 11)] and reasons[(3, 0)] == "eos"
    done = [e for e in events if e.kind == "done"][0]
    assert done.tokens == 2


def test_a_row_without_a_token_ends_its_request_with_an_error():
    """The sampler reports a row whose logits named no token (none finite) as a negative id: that
    request ends with ``invalid_logits``, nothing is emitted for the row, the others go on, and
    with the loop one step ahead the step already booked for the request is dropped."""
    for ahead in (False, True):
        s = Scheduler(cache(), max_batch_tokens=64, ignore_eos=True)
        s.add(Request(0, list(range(10, 20)), 6))
        s.add(Request(1, list(range(10, 25)), 6))
        out, reasons, in_flight = {0: [], 1: []}, {}, None
        for step in range(40):
            if s.idle() and in_flight is None:
                break
            plan = s.plan()
            for e in plan.entries:
                assert s.cache.grow(e.seq.seat, e.start + len(e.tokens))
            sampled = [-1 if (e.seq.request.id == 0 and e.start + len(e.tokens) == 12) else
                       fake_token(e.seq.request.id, e.start + len(e.tokens)) for e in plan.entries if e.sample]
            evs = []
            if ahead:
                launched = (s.book(plan), sampled) if plan.entries else None
                if in_flight:
                    evs = s.resolve(*in_flight)
                in_flight = launched
            else:
                evs = s.complete(plan, sampled)
            for ev in evs + plan.events:
                if ev.kind == "token":
                    out[ev.request_id].append(ev.token)
                elif ev.kind == "done":
                    reasons[ev.request_id] = (ev.reason, ev.tokens)
            s.cache.check()
        assert reasons == {0: ("invalid_logits", 2), 1: ("length", 6)}
        assert out[0] == [fake_token(0, 10), fake_token(0, 11)] and len(out[1]) == 6
        assert s.idle() and s.cache.free_seats == 8 and s.cache.groups[0].free_pages() == 64


def test_cancelling_a_request_gives_back_what_it_holds_wherever_it_is():
    s = Scheduler(cache(pages=8, seqs=2), max_batch_tokens=64, chunk_size=16, ignore_eos=True)
    s.add(Request(0, list(range(10, 50)), 9))          # will be part-way through its prompt
    s.add(Request(1, list(range(10, 20)), 9))          # will be decoding
    s.add(Request(2, list(range(10, 20)), 9))          # waits for a seat
    for _ in range(2):
        plan = s.plan()
        for e in plan.entries:
            assert s.cache.grow(e.seq.seat, e.start + len(e.tokens))
        s.complete(plan, [fake_token(e.seq.request.id, e.start + len(e.tokens)) for e in plan.entries if e.sample])
    assert [q.request.id for q in s.running] == [0, 1] and s.running[0].prefilling and not s.running[1].prefilling
    # a step booked but not resolved: the token it will bring for request 1 is dropped
    plan = s.plan()
    for e in plan.entries:
        assert s.cache.grow(e.seq.seat, e.start + len(e.tokens))
    ticket = s.book(plan)
    evs = s.cancel(1) + s.cancel(2) + s.cancel(7)       # decoding, waiting, unknown
    assert [(e.kind, e.request_id, e.reason, e.tokens) for e in evs] == [("done", 1, "cancelled", 2), ("done", 2, "cancelled", 0)]
    sampled = [fake_token(e.seq.request.id, e.start + len(e.tokens)) for e in plan.entries if e.sample]
    assert all(ev.request_id == 0 for ev in s.resolve(ticket, sampled))
    s.cache.check()
    assert s.cache.free_seats == 1 and not s.waiting
    out, reasons, _, _ = run(s)
    assert reasons == {(0, 0): "length"} and len(out[(0, 0)]) in (8, 9)
    assert s.cache.free_seats == 2 and s.cache.groups[0].free_pages() == 8


def test_n_seqs_share_an_id_and_differ_by_seq_index():
    s = Scheduler(cache(), ignore_eos=True)
    for i in range(3):
        s.add(Request(5, [9, 9, 9], 4, seq_index=i))
    out, reasons, _, _ = run(s)
    assert sorted(out) == [(5, 0), (5, 1), (5, 2)] and all(len(v) == 4 for v in out.values())


def test_pages_run_out_newest_is_preempted_recomputed_and_emits_nothing_twice():
    def go(pages):
        s = Scheduler(cache(pages=pages), max_batch_tokens=256, ignore_eos=True)
        for i in range(3):
            s.add(Request(i, [8 + i] * 30, 60))       # each ends at 90 tokens = 6 pages
        return s, run(s)
    s_big, (out_big, _, ev_big, _) = go(64)
    s_small, (out_small, reasons, ev_small, plans) = go(12)   # 3 x 6 pages do not fit
    assert s_big.preemptions == 0 and s_small.preemptions > 0
    assert out_small == out_big                        # identical tokens, none emitted twice
    pre = [e for e in ev_small if e.kind == "preempted"]
    assert pre and pre[0].request_id == 2 and pre[0].reason == "recompute"   # the newest goes first
    assert all(r == "length" for r in reasons.values())
    # the preempted request re-enters at the FRONT and is admitted before anything newer
    assert s_small.cache.groups[0].free_pages() == 12 and not s_small.preemption_pending


def test_admission_is_closed_to_new_requests_while_a_preempted_one_is_pending():
    s = Scheduler(cache(pages=8), max_batch_tokens=256, ignore_eos=True)
    s.add(Request(0, [9] * 40, 50))                   # ends at 90 tokens = 6 pages
    s.add(Request(1, [9] * 40, 50))
    seen_new_while_pending = []

    def watch(plan):
        if s.preemption_pending:
            seen_new_while_pending.extend(e.seq.request.id for e in plan.entries if e.seq.request.id == 2)
    s.plan_calls = 0
    steps = 0
    while not s.idle():
        plan = s.plan()
        if steps == 3:
            s.add(Request(2, [9] * 10, 5))             # a fresh request arrives
        watch(plan)
        for e in plan.entries:
            assert s.cache.grow(e.seq.seat, e.start + len(e.tokens))
        s.complete(plan, [fake_token(e.seq.request.id, e.start + len(e.tokens)) for e in plan.entries if e.sample])
        s.cache.check()
        steps += 1
        assert steps < 2000
    assert s.preemptions > 0 and not seen_new_while_pending


def test_hopeless_requests_fail_loudly_instead_of_waiting_forever():
    s = Scheduler(cache(pages=4, max_len=512), ignore_eos=True)
    s.add(Request(0, [9] * 100, 5))                   # 7 pages, the pool has 4
    s.add(Request(1, [9] * 600, 5))                   # longer than the longest sequence
    s.add(Request(2, [], 5))
    s.add(Request(3, [9] * 20, 100))                  # fits at first, outgrows the pool alone
    out, reasons, _, _ = run(s)
    assert reasons[(0, 0)] == "kv_cache_exhausted" and reasons[(1, 0)] == "prompt_too_long"
    assert reasons[(2, 0)] == "empty_request" and reasons[(3, 0)] == "kv_cache_exhausted"
    assert len(out[(3, 0)]) == 4 * 16 - 20 + 1        # it ran until the pool was full
    assert s.cache.groups[0].free_pages() == 4


def test_a_request_stops_at_the_longest_sequence():
    s = Scheduler(cache(max_len=40), ignore_eos=True)
    s.add(Request(0, [9] * 30, 100))
    out, reasons, _, _ = run(s)
    assert reasons[(0, 0)] == "sequence_too_long" and len(out[(0, 0)]) == 11


def test_reservation_policies_are_the_papers():
    assert reservation_tokens("max", 40, 25, 2048) == 2048
    assert reservation_tokens("pow2", 40, 25, 2048) == 72         # 40 + 32, reference engine.cu:314-317
    assert reservation_tokens("pow2", 0, 25, 2048) == 32          # reference config.h:192-195
    assert reservation_tokens("oracle", 40, 25, 2048) == 65
    assert reservation_tokens("oracle", 2000, 100, 2048) == 2048
    with pytest.raises(ValueError):
        reservation_tokens("best", 1, 1, 1)


def test_contiguous_mode_blocks_at_the_head_never_preempts_and_stops_at_the_reservation():
    s = Scheduler(cache(pages=16, mode="contiguous", max_len=128), reserve_policy="oracle",
                  max_batch_tokens=256, ignore_eos=True)
    s.add(Request(0, [9] * 60, 60))                   # 120 tokens -> 8 pages
    s.add(Request(1, [9] * 60, 60))                   # 8 pages
    s.add(Request(2, [9] * 10, 5))                    # waits behind the full pool
    p = s.plan()
    assert [e.seq.request.id for e in p.entries] == [0, 1] and len(s.waiting) == 1
    s.complete(p, [fake_token(0, 60), fake_token(1, 60)])
    out, reasons, _, _ = run(s)
    assert s.preemptions == 0 and all(r == "length" for r in reasons.values()) and len(out[(2, 0)]) == 5
    # under 'max' every request takes the longest sequence: only one fits at a time
    s = Scheduler(cache(pages=8, mode="contiguous", max_len=128), reserve_policy="max", ignore_eos=True)
    for i in range(3):
        s.add(Request(i, [9] * 10, 3))
    out, reasons, _, plans = run(s)
    assert max(len(p.entries) for p in plans) == 1 and len(out) == 3
    # a reservation that is used up ends the request
    s = Scheduler(cache(pages=16, mode="contiguous", max_len=64), reserve_policy="max", ignore_eos=True)
    s.add(Request(0, [9] * 60, 100))
    out, reasons, _, _ = run(s)
    assert reasons[(0, 0)] == "sequence_too_long" and len(out[(0, 0)]) == 5


# ----------------------------------------------------------------------------------------------
# Running ahead: a step is booked before its tokens are known and resolved one step later.

def run_ahead(s, max_steps=10000):
    """Like ``run``, but the tokens of a step reach the scheduler only after the NEXT step has been
    planned and booked, and a decode entry may name its token by feedback row."""
    from kv_cache_optimization_for_llm_amd.engine.scheduler import UnresolvedTokens
    out, reasons, events = {}, {}, []
    in_flight = None                       # (ticket, sampled values)
    resolved_early = 0
    feedback = []                          # what "the device" holds: the last sampling's tokens

    def resolve():
        nonlocal in_flight
        evs = s.resolve(*in_flight) if in_flight else []
        in_flight = None
        return evs

    for _ in range(max_steps):
        if s.idle() and in_flight is None:
            break
        evs = []
        try:
            plan = s.plan()
        except UnresolvedTokens:
            resolved_early += 1
            evs += resolve()
            plan = s.plan()
        s.cache.check()
        launched = None
        if plan.entries:
            sampled = []
            for e in plan.entries:
                assert s.cache.grow(e.seq.seat, e.start + len(e.tokens)), "the plan promised pages it cannot get"
                toks = [feedback[-1 - t] if t < 0 else t for t in e.tokens]
                if len(e.tokens) == 1 and e.start >= len(e.seq.prompt):
                    # a decoded token is the one "the model" sampled for this position
                    assert toks[0] == fake_token(e.seq.request.id, e.start), "a stale feedback row was named"
                assert all(t >= 0 for t in toks[1:]) and (toks[0] >= 0)
                if e.sample:
                    sampled.append(fake_token(e.seq.request.id, e.start + len(e.tokens)))
            launched = (s.book(plan), sampled)
            feedback = sampled
        evs += resolve()
        evs += plan.events
        in_flight = launched
        s.cache.check()
        for ev in evs:
            key = (ev.request_id, ev.seq_index)
            if ev.kind == "token":
                out.setdefault(key, []).append(ev.token)
            elif ev.kind in ("done", "rejected"):
                assert key not in reasons, "a request finished twice"
                reasons[key] = ev.reason
        events += evs
    assert s.idle() and in_flight is None, "the scheduler did not finish"
    return out, reasons, events, resolved_early


def eos_position(request_id, start, limit=400):
    for p in range(start, limit):
        if fake_token(request_id, p) == EOS + 8:
            return p
    return None


@pytest.mark.parametrize("pages", [64, 8])
def test_running_ahead_gives_the_tokens_and_reasons_of_the_synchronous_loop(pages):
    """Same requests, same made-up model: booking a step before its tokens are seen changes when
    things are known, not what is emitted - with end-of-sequence tokens (a token computed for a
    request that had already ended is dropped) and, with few pages, preemptions (which wait for
    the values)."""
    eos = EOS + 8                                     # a value fake_token does produce
    lens = [5, 17, 33, 40, 1, 9, 21]

    def make():
        s = Scheduler(cache(pages=pages, seqs=4), max_batch_tokens=48, chunk_size=16, eos_token_ids=[eos])
        for i, n in enumerate(lens):
            s.add(Request(i, [20 + (j % 50) for j in range(n)], 30 + i))
        return s

    want_out, want_reasons, _, _ = run(make())
    s = make()
    out, reasons, events, early = run_ahead(s)
    assert out == want_out and reasons == want_reasons
    assert any(r == "eos" for r in reasons.values()) and any(r == "length" for r in reasons.values())
    if pages == 8:
        assert s.preemptions > 0 and early > 0
    assert all(g.free_pages() == g.num_pages for g in s.cache.groups) and s.cache.free_seats == 4


def test_planning_refuses_to_preempt_while_tokens_are_unseen_and_changes_nothing():
    from kv_cache_optimization_for_llm_amd.engine.scheduler import UnresolvedTokens
    s = Scheduler(cache(pages=4, seqs=4), max_batch_tokens=64, ignore_eos=True)
    s.add(Request(0, list(range(8, 8 + 31)), 40))
    s.add(Request(1, list(range(8, 8 + 31)), 40))
    p = s.plan()                                       # both prompts: 2 pages each, pool is full
    for e in p.entries:
        assert s.cache.grow(e.seq.seat, e.start + len(e.tokens))
    t1 = s.book(p)
    p2 = s.plan()                                      # position 31 still fits the second page
    assert [e.tokens for e in p2.entries] == [[-1], [-2]]
    for e in p2.entries:
        assert s.cache.grow(e.seq.seat, e.start + 1)
    s.resolve(t1, [fake_token(0, 31), fake_token(1, 31)])
    t2 = s.book(p2)
    before = (len(s.running), len(s.waiting), s.preemptions, [g.free_pages() for g in s.cache.groups])
    with pytest.raises(UnresolvedTokens):
        s.plan()                                       # position 32 needs a third page each: none free
    assert before == (len(s.running), len(s.waiting), s.preemptions, [g.free_pages() for g in s.cache.groups])
    evs = s.resolve(t2, [fake_token(0, 32), fake_token(1, 32)])
    assert [e.kind for e in evs] == ["token", "token"]
    p3 = s.plan()
    assert [e.kind for e in p3.events] == ["preempted"] and p3.events[0].request_id == 1
    assert s.waiting[0].tokens[-2:] == [fake_token(1, 31), fake_token(1, 32)]


def test_prompts_admitted_together_are_counted_with_the_pages_they_still_need():
    """Two seats, 32 pages of 4 tokens, portions of 8: a prompt is mapped portion by portion, so
    the pages free at admission are not all free for a second newcomer.  Prompts of 84 and 58
    tokens (36 pages) must not both be admitted - they would stop half-way with no page left and
    nothing to give one back."""
    s = Scheduler(cache(pages=32, seqs=2, page=4, max_len=101), max_batch_tokens=64, chunk_size=8, ignore_eos=True)
    lens = [63, 57, 12, 28, 84, 58, 16, 53]
    for i, n in enumerate(lens):
        s.add(Request(i, [8 + (j % 30) for j in range(n)], 16))
    out, reasons, events, plans = run(s, max_steps=2000)
    for i, n in enumerate(lens):
        assert reasons[(i, 0)] == "length" and out[(i, 0)] == [fake_token(i, n + k) for k in range(16)]
    for p in plans:
        assert p.entries or p.events, "a plan with nothing to run and nothing to report"


@pytest.mark.parametrize("policy", ["max", "pow2", "oracle"])
def test_running_ahead_in_contiguous_mode_makes_the_head_wait_for_a_closing_request(policy):
    """Three equal requests, a pool for two reservations of the longest sequence: the third has to
    wait, also while the two before it only wait for their last token's value (they hold their
    runs one step longer when the loop runs ahead).  The reference's queue head blocks until its
    reservation can be placed and nothing that fits is refused (``base/src/engine.cu:432-437``)."""
    def make():
        s = Scheduler(cache(pages=16, seqs=4, mode="contiguous", max_len=128), reserve_policy=policy,
                      max_batch_tokens=64, ignore_eos=True)
        for i in range(3):
            s.add(Request(i, [9] * 10, 3))
        return s
    want_out, want_reasons, _, _ = run(make())
    assert all(r == "length" for r in want_reasons.values()) and len(want_reasons) == 3
    s = make()
    out, reasons, _, _ = run_ahead(s)
    assert out == want_out and reasons == want_reasons
    assert s.preemptions == 0 and s.cache.free_seats == 4


@pytest.mark.parametrize("policy", ["max", "pow2", "oracle"])
@pytest.mark.parametrize("seed", range(12))
def test_running_ahead_gives_the_synchronous_loops_results_in_contiguous_mode(seed, policy):
    """Random requests with end-of-sequence tokens on a pool that holds two or three reservations:
    the same tokens and the same reasons from both loops, and a request is failed only if its
    reservation cannot be placed in an empty pool."""
    import numpy as np
    rng = np.random.default_rng(1000 + seed)
    eos = EOS + 8
    lens = [int(x) for x in rng.integers(1, 60, int(rng.integers(3, 9)))]
    news = [int(x) for x in rng.integers(1, 40, len(lens))]
    max_len = 128
    pages = int(rng.integers(8, 24))                    # pages of 16: 128 to 384 tokens

    def make():
        s = Scheduler(cache(pages=pages, seqs=4, mode="contiguous",
                            max_len=max_len), reserve_policy=policy, max_batch_tokens=48,
                      chunk_size=16, eos_token_ids=[eos])
        for i, (n, k) in enumerate(zip(lens, news)):
            s.add(Request(i, [20 + (j % 50) for j in range(n)], k))
        return s

    want_out, want_reasons, _, _ = run(make())
    s = make()
    out, reasons, _, _ = run_ahead(s)
    assert out == want_out and reasons == want_reasons
    assert set(want_reasons.values()) <= {"length", "eos", "sequence_too_long"}
    assert s.preemptions == 0 and s.cache.free_seats == 4
    s.cache.check()


@pytest.mark.parametrize("mode", ["paged", "contiguous"])
@pytest.mark.parametrize("ahead", [False, True])
@pytest.mark.parametrize("seed", range(40))
def test_random_tight_pools_always_finish(seed, ahead, mode):
    """Random prompts, budgets, portion sizes, page sizes and pools barely larger than the longest
    request: every request ends, with its full budget of the right tokens unless the cache
    could not hold it, and no page is lost.  In contiguous mode a request reserves a power-of-two
    run of pages; one whose run is larger than the largest the pool can ever place fails alone, in
    both loops alike, and every other gets its full budget."""
    import numpy as np
    rng = np.random.default_rng(seed)
    page = int(rng.choice([16, 8, 4]))
    lens = [int(x) for x in rng.integers(1, 90, int(rng.integers(3, 9)))]
    new = int(rng.integers(4, 20))
    seats = int(rng.integers(2, 5))
    longest = max(lens) + new + 1
    pool = int(rng.integers(longest + page, seats * longest + 2 * page))
    chunk = int(rng.choice([0, 8, 24, 64])) or None
    policy = str(rng.choice(["max", "pow2", "oracle"]))
    s = Scheduler(cache(pages=(pool + page - 1) // page, seqs=seats, page=page, max_len=longest, mode=mode),
                  max_batch_tokens=int(rng.choice([32, 64, 256])), chunk_size=chunk, ignore_eos=True,
                  reserve_policy=policy)
    for i, n in enumerate(lens):
        s.add(Request(i, [8 + (j % 30) for j in range(n)], new))
    out, reasons, events, plans = (run_ahead if ahead else run)(s, max_steps=4000)
    for i, n in enumerate(lens):
        if mode == "contiguous":
            # what the request reserves, as a run of pages rounded up to a power of two, against
            # the largest run an empty pool of this size holds
            run_pages = -(-reservation_tokens(policy, n, new, longest) // page)
            run_pages = 1 << (run_pages - 1).bit_length()
            pool_pages = (pool + page - 1) // page
            if run_pages > 1 << (pool_pages.bit_length() - 1):
                assert reasons[(i, 0)] == "kv_cache_exhausted" and (i, 0) not in out, (i, reasons)
                continue
        assert reasons[(i, 0)] == "length", (i, reasons)
        assert out[(i, 0)] == [fake_token(i, n + k) for k in range(new)]
    s.cache.check()
    assert s.cache.free_seats == seats


def test_admission_asks_each_group_what_a_prompt_needs():
    """A group that keeps only a window of keys needs a window's worth of pages however long the
    prompt is; a model without keys needs none.  Admission by ceil(prompt / page) for every
    group would refuse (or make wait) requests that fit."""
    from kv_cache_optimization_for_llm_amd.parts.base import StateSpec
    win = attention_cache_spec(1, 16, kind="window", window=20)
    # 6 pages of 16: a prompt of 300 tokens is 19 pages of keys, but 20 - 1 + 16 positions at a time
    m = CacheManager([(win, [0])], {}, page_size=16, num_pages=6, max_seqs=2, max_seq_len=512)
    g = m.groups[0]
    assert g.pages_for(300) == 19 and g.pages_for(300, 16) == 4 and g.pages_for(10, 16) == 1
    assert CacheManager([(SPEC, [0])], {}, page_size=16, num_pages=6, max_seqs=2,
                        max_seq_len=512).groups[0].pages_for(300, 16) == 19
    s = Scheduler(m, max_batch_tokens=64, chunk_size=16, ignore_eos=True)
    s.add(Request(0, list(range(8, 308)), 4))
    s.add(Request(1, list(range(8, 40)), 4))
    out, reasons, events, plans = run(s)
    assert reasons == {(0, 0): "length", (1, 0): "length"} and len(out[(0, 0)]) == 4
    assert not any(e.kind == "preempted" for e in events)
    assert max(len(p.entries) for p in plans) == 2                # both were live together
    assert g.free_pages() == 6 and g.pool.reuses > 0
    # all keys kept: the same prompt cannot be held by 6 pages and fails alone, as before
    full = CacheManager([(SPEC, [0])], {}, page_size=16, num_pages=6, max_seqs=2, max_seq_len=512)
    s = Scheduler(full, max_batch_tokens=64, chunk_size=16, ignore_eos=True)
    s.add(Request(0, list(range(8, 308)), 4))
    assert run(s)[1] == {(0, 0): "kv_cache_exhausted"}
    # no group at all (a model that keeps a fixed-size state per request): seats are the only limit
    none = CacheManager([], {0: StateSpec((4,))}, page_size=16, num_pages=1, max_seqs=2, max_seq_len=512)
    s = Scheduler(none, max_batch_tokens=64, chunk_size=16, ignore_eos=True)
    for i in range(3):
        s.add(Request(i, list(range(8, 108)), 3))
    out, reasons, _, plans = run(s)
    assert reasons == {(i, 0): "length" for i in range(3)} and all(len(v) == 3 for v in out.values())


@pytest.mark.parametrize("multiple, chunk, budget", [(8, 20, 50), (5, 5, 17), (16, 64, 40), (3, 100, 29)])
def test_portions_end_where_the_mixers_can_be_cut(multiple, chunk, budget):
    """A model whose mixers take a prompt only in portions that end on multiples of so many
    positions: every portion but a prompt's last ends there, whatever the token budget and the
    other requests leave, and every request still emits all its tokens."""
    s = Scheduler(cache(pages=128), max_batch_tokens=budget, chunk_size=chunk, ignore_eos=True,
                  portion_multiple=multiple)
    lengths = [1, multiple - 1, multiple, multiple + 1, 61, 100, 37]
    for i, n in enumerate(lengths):
        s.add(Request(i, [8 + (j % 50) for j in range(n)], 6))
    cuts = []

    def watch(plan):
        assert plan.num_tokens <= budget
        for e in plan.entries:
            if len(e.tokens) > 1 or e.start < len(e.seq.prompt):
                end = e.start + len(e.tokens)
                assert e.start % multiple == 0 and (end % multiple == 0 or end == len(e.seq.prompt)), (e.start, end)
                cuts.append((e.seq.request.id, e.start, end))
    out, reasons, _, _ = run(s, on_plan=watch)
    assert all(len(out[(i, 0)]) == 6 and reasons[(i, 0)] == "length" for i in range(len(lengths)))
    assert any(end % multiple == 0 and end < lengths[i] for i, _, end in cuts), "no prompt was cut at all"


def test_a_portion_multiple_that_cannot_be_kept_is_refused():
    with pytest.raises(ValueError):
        Scheduler(cache(), max_batch_tokens=16, portion_multiple=32)
    with pytest.raises(ValueError):
        Scheduler(cache(), max_batch_tokens=64, chunk_size=8, portion_multiple=16)
    with pytest.raises(ValueError):
        Scheduler(cache(), max_batch_tokens=64, portion_multiple=0)
