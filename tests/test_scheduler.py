"""The scheduler's decisions, the request state machine and the engine loop (no GPU)."""

from __future__ import annotations

import random

import pytest
from fake_runner import ArgmaxSampler, FakeRunner, expected_generation

from miniserve_amd.cache import CapacitySnapshot
from miniserve_amd.config import EngineConfig
from miniserve_amd.engine import (
    DecodeItem,
    Engine,
    ExecutionPlan,
    PrefillItem,
    Request,
    RequestStatus,
    SamplingParams,
    Scheduler,
    SequenceState,
    SequenceView,
)

W, P, D = RequestStatus.WAITING, RequestStatus.PREFILLING, RequestStatus.DECODING


def view(name, status, *, target=10, cursor=0, generated=0, arrival=0, max_new=8) -> SequenceView:
    computed = cursor if status is not D else target + generated - 1
    total = target if status is not D else target + generated
    return SequenceView(
        request_id=name, status=status, prefill_target=target, computed_tokens=computed, total_tokens=total, num_generated=generated, max_new_tokens=max_new,
        arrival_ns=arrival, next_input_token_id=7 if status is D else None,
    )


def capacity(free, *, total=64, block_size=4, free_slots=4, slots=8, held=None) -> CapacitySnapshot:
    return CapacitySnapshot((block_size,), (total,), (free,), free_slots, slots, held or {})


def scheduler(**options) -> Scheduler:
    base = dict(max_num_seqs=8, max_num_batched_tokens=32)
    base.update(options)
    return Scheduler(**base)


# ---- the request state machine: the reference's vectors --------------------------------

def request(max_new_tokens=2, stop=()):
    return Request("r", (10, 20, 30), SamplingParams(max_new_tokens=max_new_tokens, stop_token_ids=stop), 1)


def test_prefill_and_decode_preserve_pending_token_invariant():
    # reference: tests/unit/test_sequence_state.py:54-71
    state = SequenceState.from_request(request())
    state.admitted()
    state.ran_to(3)
    state.take_token(42)
    assert state.status is D and state.all_tokens == (10, 20, 30, 42)
    assert state.computed_tokens == 3 and state.total_tokens == state.computed_tokens + 1
    assert state.snapshot().next_input_token_id == 42
    state.ran_pending_token()
    state.take_token(43)
    assert state.ending() == "length"
    state.finish("length")
    assert state.status is RequestStatus.FINISHED and state.computed_tokens == state.total_tokens - 1


def test_tokens_are_read_without_building_the_whole_sequence():
    state = SequenceState.from_request(request(max_new_tokens=4))
    state.admitted()
    state.ran_to(3)
    for token in (42, 43):
        state.take_token(token)
        state.ran_pending_token()
    state.take_token(44)
    everything = state.all_tokens
    assert everything == (10, 20, 30, 42, 43, 44)
    assert [state.token_at(i) for i in range(6)] == list(everything)
    for start in range(6):
        for end in range(start + 1, 7):
            assert state.tokens_between(start, end) == everything[start:end]


def test_stop_token_finishes_without_being_run():
    # reference: tests/unit/test_sequence_state.py:74-82
    state = SequenceState.from_request(request(max_new_tokens=4, stop=(99,)))
    state.admitted()
    state.ran_to(3)
    state.take_token(99)
    assert state.ending() == "stop"
    state.finish("stop")
    assert state.computed_tokens == 3 and state.total_tokens == 4


def test_partial_prefill_does_not_sample_and_illegal_moves_fail():
    # reference: tests/unit/test_sequence_state.py:84-104
    state = SequenceState.from_request(request())
    with pytest.raises(RuntimeError, match="only a DECODING request can run its pending token"):
        state.ran_pending_token()
    state.admitted()
    state.ran_to(2)
    assert state.status is P and state.computed_tokens == 2
    with pytest.raises(RuntimeError, match="a token is sampled only after all of them"):
        state.take_token(1)
    with pytest.raises(RuntimeError, match="does not move it forward"):
        state.ran_to(2)
    state.ran_to(3)
    state.take_token(42)
    assert state.status is D


def test_preemption_keeps_tokens_and_runs_them_again():
    state = SequenceState.from_request(request(max_new_tokens=5))
    state.admitted()
    state.ran_to(3)
    state.take_token(42)
    state.ran_pending_token()
    state.take_token(43)
    state.preempt()
    snapshot = state.snapshot()
    assert snapshot.status is W and snapshot.prefill_target == 5 and snapshot.computed_tokens == 0
    assert snapshot.num_generated == 2 and snapshot.num_preemptions == 1
    state.admitted()
    state.ran_to(5)
    state.take_token(44)
    assert state.all_tokens == (10, 20, 30, 42, 43, 44) and state.status is D


def test_plan_checks():
    # reference: tests/unit/test_sequence_state.py:107-138
    ExecutionPlan(0, (PrefillItem("r", 0, 3),), (), 3)
    with pytest.raises(ValueError, match="its items hold"):
        ExecutionPlan(2, (PrefillItem("r", 0, 2),), (), 1)
    with pytest.raises(TypeError, match="takes tuples"):
        ExecutionPlan(0, [PrefillItem("r", 0, 1)], (), 1)
    with pytest.raises(ValueError, match="more than once"):
        ExecutionPlan(0, (PrefillItem("r", 0, 1),), (DecodeItem("r", 1, 1),), 2)
    with pytest.raises(ValueError, match="preempted and run in the same step"):
        ExecutionPlan(0, (PrefillItem("r", 0, 1),), (), 1, preempted=("r",))
    for invalid in (True, 1.5):
        with pytest.raises(ValueError):
            DecodeItem("r", invalid, 0)


# ---- decisions -------------------------------------------------------------------------

def test_decode_first_then_prompts_in_arrival_order():
    views = [
        view("late-waiting", W, arrival=5, target=6),
        view("decoding-b", D, arrival=2, generated=1),
        view("early-waiting", W, arrival=3, target=9),
        view("decoding-a", D, arrival=1, generated=2),
    ]
    plan = scheduler().schedule(views, capacity(40))
    assert [i.request_id for i in plan.decode_items] == ["decoding-a", "decoding-b"]
    assert plan.decode_items[0].position == 11 and plan.decode_items[0].input_token_id == 7
    assert [(i.request_id, i.token_start, i.token_end) for i in plan.prefill_items] == [
        ("early-waiting", 0, 9), ("late-waiting", 0, 6),
    ]
    assert plan.scheduled_tokens == 17 and plan.preempted == ()


def test_same_arrival_is_ordered_by_id_and_the_function_is_pure():
    views = [view("b", W, target=20), view("a", W, target=20)]
    first = scheduler(max_num_batched_tokens=25).schedule(views, capacity(40))
    second = scheduler(max_num_batched_tokens=25).schedule(list(reversed(views)), capacity(40))
    assert first == second
    assert [i.request_id for i in first.prefill_items] == ["a"]      # whole prompts only: b does not fit


def test_token_budget_and_portions():
    views = [view("a", W, target=50), view("b", W, arrival=1, target=10)]
    whole = scheduler().schedule(views, capacity(40))
    assert [(i.request_id, i.token_end) for i in whole.prefill_items] == [("b", 10)]   # a never fits unchunked
    chunked = scheduler(enable_chunked_prefill=True).schedule(views, capacity(40))
    assert [(i.request_id, i.token_start, i.token_end) for i in chunked.prefill_items] == [("a", 0, 32)]
    sized = scheduler(enable_chunked_prefill=True, prefill_chunk_size=7).schedule(views, capacity(40))
    assert [(i.request_id, i.token_end) for i in sized.prefill_items] == [("a", 7), ("b", 7)]
    resumed = scheduler(enable_chunked_prefill=True, prefill_chunk_size=7).schedule(
        [view("a", P, target=50, cursor=49)], capacity(40)
    )
    assert [(i.token_start, i.token_end) for i in resumed.prefill_items] == [(49, 50)]   # a portion of one token


def test_decoding_cannot_starve_a_prompt_when_portions_are_allowed():
    # reference: miniserve/engine/scheduler.py:150-164
    views = [view(f"d{i}", D, arrival=i, generated=1) for i in range(4)] + [view("p", W, arrival=9, target=30)]
    plan = scheduler(max_num_batched_tokens=4, enable_chunked_prefill=True).schedule(views, capacity(40))
    assert len(plan.decode_items) == 3 and [(i.request_id, i.token_end) for i in plan.prefill_items] == [("p", 1)]
    plain = scheduler(max_num_batched_tokens=4).schedule(views, capacity(40))
    assert len(plain.decode_items) == 4 and plain.prefill_items == ()


def test_portion_shrinks_to_the_pages_that_are_free():
    # 2 free pages of 4 and 1 token of room in the request's last page
    plan = scheduler(enable_chunked_prefill=True).schedule([view("a", P, target=40, cursor=7)], capacity(2))
    assert [(i.token_start, i.token_end) for i in plan.prefill_items] == [(7, 16)]
    none = scheduler(enable_chunked_prefill=True).schedule([view("a", W, target=40)], capacity(0))
    assert none.empty
    whole = scheduler().schedule([view("a", W, target=40)], capacity(2))
    assert whole.empty                                            # whole prompts are not cut


def test_waiting_requests_need_a_state_slot():
    views = [view("a", W, target=4), view("b", W, arrival=1, target=4)]
    plan = scheduler().schedule(views, capacity(40, free_slots=1))
    assert [i.request_id for i in plan.prefill_items] == ["a"]
    capped = scheduler(max_num_seqs=2).schedule([view("x", D, generated=1), view("y", D, arrival=1, generated=1)] + views,
                                                capacity(40, free_slots=3))
    assert capped.prefill_items == ()


def test_out_of_pages_preempts_the_youngest_running_request():
    # every request stands at a page edge (computed 12 = 3 pages of 4) and needs a new page; none is free
    views = [view(n, D, arrival=i, target=10, generated=3) for i, n in enumerate(("old", "mid", "young"))]
    held = {"old": (3,), "mid": (3,), "young": (3,)}
    plan = scheduler().schedule(views, capacity(0, held=held))
    assert plan.preempted == ("young",)
    assert [i.request_id for i in plan.decode_items] == ["old", "mid"]
    # with one free page nobody is preempted but the last one in line waits
    plan = scheduler().schedule(views, capacity(1, held=held))
    assert plan.preempted == ("young",) and [i.request_id for i in plan.decode_items] == ["old", "mid"]
    plan = scheduler().schedule(views, capacity(3, held=held))
    assert plan.preempted == () and len(plan.decode_items) == 3


def test_the_oldest_is_never_preempted_and_waiting_requests_preempt_nobody():
    alone = [view("old", D, target=10, generated=3)]
    plan = scheduler().schedule(alone, capacity(0, held={"old": (3,)}))
    assert plan.preempted == () and plan.empty                      # it waits; nothing younger exists
    views = [view("run", D, arrival=5, target=10, generated=3), view("new", W, arrival=0, target=8)]
    plan = scheduler().schedule(views, capacity(1, held={"run": (3,)}))
    assert plan.preempted == () and [i.request_id for i in plan.decode_items] == ["run"]
    assert plan.prefill_items == ()                                  # no page left for the older waiting request


def test_a_prompt_in_progress_may_preempt_a_younger_one_but_not_one_already_scheduled():
    views = [view("older", P, arrival=0, target=40, cursor=8), view("younger", P, arrival=1, target=40, cursor=8)]
    held = {"older": (2,), "younger": (2,)}
    plan = scheduler(enable_chunked_prefill=True, prefill_chunk_size=8).schedule(views, capacity(0, held=held))
    assert plan.preempted == ("younger",)
    assert [(i.request_id, i.token_start, i.token_end) for i in plan.prefill_items] == [("older", 8, 16)]
    views = [view("older", P, arrival=0, target=40, cursor=8), view("younger", D, arrival=1, target=7, generated=1)]
    plan = scheduler(enable_chunked_prefill=True, prefill_chunk_size=8).schedule(views, capacity(0, held=held))
    assert plan.preempted == () and [i.request_id for i in plan.decode_items] == ["younger"]
    assert plan.prefill_items == ()


@pytest.mark.parametrize("seed", range(5))
def test_budgets_hold_for_random_views(seed):
    rng = random.Random(seed)
    for _ in range(60):
        views, held = [], {}
        for index in range(rng.randint(1, 9)):
            status = rng.choice((W, P, D))
            target = rng.randint(1, 40)
            cursor = 0 if status is W else (rng.randint(1, target) - 1 if status is P else target)
            generated = rng.randint(1, 5) if status is D else 0
            v = view(f"r{index}", status, target=target, cursor=cursor, generated=generated, arrival=rng.randint(0, 4))
            views.append(v)
            if status is not W:
                held[v.request_id] = (-(-v.computed_tokens // 4),)
        free = rng.randint(0, 12)
        budget = rng.randint(1, 24)
        chunked = rng.random() < 0.5
        running = sum(1 for v in views if v.status is not W)
        plan = Scheduler(max_num_seqs=8, max_num_batched_tokens=budget, enable_chunked_prefill=chunked).schedule(
            views, capacity(free, free_slots=8 - running, held=held)
        )
        assert plan.scheduled_tokens <= budget
        by_id = {v.request_id: v for v in views}
        pages = sum(held[r][0] for r in plan.preempted) + free
        for item in plan.decode_items:
            v = by_id[item.request_id]
            pages -= -(-(v.computed_tokens + 1) // 4) - -(-v.computed_tokens // 4)
        for item in plan.prefill_items:
            v = by_id[item.request_id]
            assert item.token_start == v.computed_tokens and item.token_end <= v.prefill_target
            if not chunked:
                assert item.token_end == v.prefill_target
            pages -= -(-item.token_end // 4) - -(-item.token_start // 4)
        assert pages >= 0
        oldest_running = min((v for v in views if v.status is not W), key=lambda v: (v.arrival_ns, v.request_id), default=None)
        if oldest_running is not None:
            assert oldest_running.request_id not in plan.preempted
        assert all(by_id[r].status is not W for r in plan.preempted)


# ---- the engine loop with a stand-in runner ---------------------------------------------

def make_engine(**options):
    base = dict(dtype="float32", kv_block_size=4, num_kv_blocks=64, max_num_seqs=4, max_model_len=128)
    base.update(options)
    fail = base.pop("fail_on_step", None)
    runner = FakeRunner(EngineConfig(**base), fail_on_step=fail)
    return Engine(runner, sampler=ArgmaxSampler()), runner


PROMPTS = [[3, 1, 4, 1, 5], list(range(17)), list(range(40, 73)), [9]]


def test_generate_is_the_same_whatever_the_scheduling():
    expected = [expected_generation(p, 12, 97) for p in PROMPTS]
    params = SamplingParams(max_new_tokens=12)
    roomy, _ = make_engine()
    assert roomy.generate(PROMPTS, params) == expected
    chunked, runner = make_engine(enable_chunked_prefill=True, prefill_chunk_size=7, max_num_batched_tokens=16)
    assert chunked.generate(PROMPTS, params) == expected
    assert any(len(step) > 1 for step in runner.steps)                 # portions ran beside decoded tokens
    # so few pages that requests are preempted and run again: 14 pages of 4 for 4 requests of up to 45 tokens
    tight, runner = make_engine(num_kv_blocks=14, enable_chunked_prefill=True, max_num_batched_tokens=64)
    assert tight.generate(PROMPTS, params) == expected
    assert tight.counters["preemptions"] > 0
    assert runner.cache.capacity().free_blocks == (14,) and runner.cache.capacity().free_slots == 4
    runner.cache.assert_invariants()


def test_decoded_tokens_run_longest_context_first():
    """The rows of single decoded tokens of a step stand first, in the order of their
    contexts, the longest first, with and without steps planned ahead; the portions of
    prompts follow in the plan's order."""

    for ahead in (False, True):
        engine, runner = make_engine(enable_chunked_prefill=True, prefill_chunk_size=8, max_num_batched_tokens=16)
        runner.prepare_ahead = ahead
        for index, prompt in enumerate(PROMPTS):
            engine.add_request(f"r{index}", prompt, SamplingParams(max_new_tokens=12), arrival_ns=index)
        decided = 0
        while engine.has_unfinished():
            before = len(runner.steps)
            engine.step()
            plan = engine.last_plan
            if plan.empty:
                continue
            assert len(runner.steps) == before + 1
            rows = runner.steps[-1]
            decoded = {item.request_id: item.position for item in plan.decode_items}
            first = rows[: len(decoded)]
            assert {request for request, _, _ in first} == set(decoded)
            starts = [start for _, start, _ in first]
            assert starts == sorted(starts, reverse=True) and all(decoded[r] == start for r, start, _ in first)
            assert [request for request, _, _ in rows[len(decoded):]] == [item.request_id for item in plan.prefill_items]
            decided += len(set(starts)) > 1 and starts != sorted(decoded.values())
        assert decided >= 5                                             # steps in which the order had something to decide


def test_steps_planned_ahead_change_no_token():
    """While a step of decoding requests runs, the next one is scheduled and its cache
    transaction opened; what the requests generate is what they generate without that,
    whatever ends it early: a stop token, a request that ends by length, a new request,
    a cancelled one, too few pages."""

    params = SamplingParams(max_new_tokens=12)
    expected = [expected_generation(p, 12, 97) for p in PROMPTS]
    engine, runner = make_engine()
    runner.prepare_ahead = True
    assert engine.generate(PROMPTS, params) == expected
    assert runner.used_ahead >= 8 and runner.discarded_ahead == 0       # all four decode together for ten steps
    assert runner.prepared_ahead == runner.used_ahead                  # the last step ends all by length: nothing to plan
    assert runner.cache.live_requests() == () and runner.cache.capacity().free_blocks == (64,)
    runner.cache.assert_invariants()

    # requests that end by length at different steps: the step after goes on without them, planned ahead
    lengths = (5, 12, 8, 10)
    engine, runner = make_engine()
    runner.prepare_ahead = True
    got = engine.generate(PROMPTS, [SamplingParams(max_new_tokens=n) for n in lengths])
    assert got == [tokens[:n] for tokens, n in zip(expected, lengths)]
    assert runner.discarded_ahead == 0 and runner.prepared_ahead == runner.used_ahead
    assert runner.used_ahead >= 9                                       # eleven decode steps, the first not foreseen
    assert runner.cache.live_requests() == () and runner.cache.capacity().free_blocks == (64,)
    runner.cache.assert_invariants()

    # a stop token ends a request inside a step that was planned ahead: the plan is dropped
    stop = expected[0][4]
    engine, runner = make_engine()
    runner.prepare_ahead = True
    got = engine.generate(PROMPTS, [SamplingParams(max_new_tokens=12, stop_token_ids=(stop,))] + [params] * 3)
    assert got[0] == expected[0][: expected[0].index(stop) + 1] and got[1:] == expected[1:]
    assert runner.discarded_ahead >= 1 and runner.used_ahead >= 4
    assert runner.cache.live_requests() == () and runner.cache.capacity().free_blocks == (64,)

    # a request that arrives, and one that is cancelled, between two steps
    engine, runner = make_engine()
    runner.prepare_ahead = True
    engine.add_request("a", PROMPTS[0], params, arrival_ns=0)
    engine.add_request("b", PROMPTS[1], params, arrival_ns=1)
    for _ in range(4):
        engine.step()
    assert runner.prepared_ahead > runner.used_ahead                   # one is waiting to be used
    engine.add_request("c", PROMPTS[3], params, arrival_ns=2)
    engine.step()                                                      # the plan ahead did not know "c"
    assert runner.discarded_ahead == 1
    for _ in range(3):
        engine.step()
    waiting = runner.prepared_ahead - runner.used_ahead - runner.discarded_ahead
    assert waiting == 1
    engine.cancel("b")                                                 # its pages go back: the open step first
    assert runner.discarded_ahead == 2
    runner.cache.assert_invariants()
    while engine.has_unfinished():
        engine.step()
    assert list(engine.pop_result("a").token_ids) == expected[0] and list(engine.pop_result("c").token_ids) == expected[3]
    assert runner.cache.live_requests() == () and runner.cache.capacity().free_blocks == (64,)

    # so few pages that decoding requests are preempted: plans ahead that would preempt are not made
    tight, runner = make_engine(num_kv_blocks=14, enable_chunked_prefill=True, max_num_batched_tokens=64)
    runner.prepare_ahead = True
    assert tight.generate(PROMPTS, params) == expected
    assert tight.counters["preemptions"] > 0
    assert runner.cache.capacity().free_blocks == (14,)
    runner.cache.assert_invariants()


def test_steps_launched_ahead_change_no_token():
    """A step of single tokens that was planned ahead is launched before the host has read
    the tokens it runs (they go from the sampling kernel to the step on the device).  The
    requests generate what they generate without that, whatever voids such a step: a stop
    token, a new request, a cancelled one, too few pages; and the tokens a launched step
    ran are the tokens the engine later says it ran (the stand-in runner checks that)."""

    def chained_engine(**options):
        engine, runner = make_engine(**options)
        engine.sampler = ArgmaxSampler(on_device=True)
        runner.prepare_ahead = runner.chain = True
        return engine, runner

    params = SamplingParams(max_new_tokens=12)
    expected = [expected_generation(p, 12, 97) for p in PROMPTS]
    engine, runner = chained_engine()
    assert engine.generate(PROMPTS, params) == expected
    # (the step behind the prompts' step runs its rows longest context first, not in the order in which that step
    # sampled them: its tokens are taken through a map of rows)
    assert runner.chained >= 8 and runner.chained == runner.used_ahead and runner.voided_chained == 0 and runner.mapped == 1
    assert runner.cache.live_requests() == () and runner.cache.capacity().free_blocks == (64,)

    # requests that end by length: the step after is planned, and launched, without them
    lengths = (5, 12, 8, 10)
    engine, runner = chained_engine()
    got = engine.generate(PROMPTS, [SamplingParams(max_new_tokens=n) for n in lengths])
    assert got == [tokens[:n] for tokens, n in zip(expected, lengths)]
    # (the step behind one in which a request ends by length has fewer rows than that one sampled: a map of rows again,
    # unless the request that ends held the last row)
    assert runner.chained == runner.used_ahead >= 9 and runner.mapped == 3
    assert runner.voided_chained == 0 and runner.discarded_ahead == 0

    # a stop token ends a request whose next token already runs: that step is thrown away
    stop = expected[0][4]
    engine, runner = chained_engine()
    got = engine.generate(PROMPTS, [SamplingParams(max_new_tokens=12, stop_token_ids=(stop,))] + [params] * 3)
    assert got[0] == expected[0][: expected[0].index(stop) + 1] and got[1:] == expected[1:]
    assert runner.voided_chained >= 1 and runner.chained > runner.voided_chained
    assert runner.cache.live_requests() == () and runner.cache.capacity().free_blocks == (64,)
    runner.cache.assert_invariants()

    # a request that arrives, and one that is cancelled, while a launched step runs
    engine, runner = chained_engine()
    engine.add_request("a", PROMPTS[0], params, arrival_ns=0)
    engine.add_request("b", PROMPTS[1], params, arrival_ns=1)
    for _ in range(4):
        engine.step()
    assert runner.prepared_ahead == runner.used_ahead + 1 and runner.chained == 4     # one runs and has not been taken yet
    engine.add_request("c", PROMPTS[3], params, arrival_ns=2)
    engine.step()                                                      # the launched step did not know "c"
    assert runner.voided_chained == 1
    for _ in range(3):
        engine.step()
    engine.cancel("b")                                                 # its pages go back: the running step first
    assert runner.voided_chained == 2
    runner.cache.assert_invariants()
    while engine.has_unfinished():
        engine.step()
    assert list(engine.pop_result("a").token_ids) == expected[0] and list(engine.pop_result("c").token_ids) == expected[3]
    assert runner.cache.live_requests() == () and runner.cache.capacity().free_blocks == (64,)

    # so few pages that decoding requests are preempted
    tight, runner = chained_engine(num_kv_blocks=14, enable_chunked_prefill=True, max_num_batched_tokens=64)
    assert tight.generate(PROMPTS, params) == expected
    assert tight.counters["preemptions"] > 0 and runner.chained > 0
    assert runner.cache.capacity().free_blocks == (14,)
    runner.cache.assert_invariants()

    # tokens that the host holds (a sampler that returns them at once) are never chained
    engine, runner = make_engine()
    runner.prepare_ahead = runner.chain = True
    assert engine.generate(PROMPTS, params) == expected and runner.chained == 0 and runner.used_ahead >= 8


def test_steps_with_prompt_portions_are_planned_ahead_too():
    """Portions of prompts beside decode tokens: the step after is foreseen as well (a
    request that is admitted in it is admitted ahead), and the steps that run are the
    very steps that run without planning ahead."""

    params = SamplingParams(max_new_tokens=12)
    expected = [expected_generation(p, 12, 97) for p in PROMPTS]
    options = dict(enable_chunked_prefill=True, prefill_chunk_size=7, max_num_batched_tokens=16, max_num_seqs=3)
    plain, plain_runner = make_engine(**options)
    assert plain.generate(PROMPTS, params) == expected
    engine, runner = make_engine(**options)
    runner.prepare_ahead = True
    assert engine.generate(PROMPTS, params) == expected
    assert runner.steps == plain_runner.steps
    assert runner.prepared_mixed >= 5 and runner.discarded_ahead == 0 and runner.prepared_ahead == runner.used_ahead
    assert runner.used_ahead >= len(runner.steps) - 3                   # all but the first step and the last ones
    assert runner.cache.live_requests() == () and runner.cache.capacity().free_blocks == (64,)
    assert runner.cache.capacity().free_slots == 3
    runner.cache.assert_invariants()

    # a stop token in a request that has just finished its prompt; a request cancelled while it waits, admitted ahead
    # (a budget of 8 tokens a step: the last request waits until the plan for the eighth step admits it)
    stop = expected[1][0]
    engine, runner = make_engine(**{**options, "max_num_batched_tokens": 8})
    runner.prepare_ahead = True
    for index, prompt in enumerate(PROMPTS):
        stops = (stop,) if index == 1 else ()
        engine.add_request(f"r{index}", prompt, SamplingParams(max_new_tokens=12, stop_token_ids=stops), arrival_ns=index)
    cancelled = False
    while engine.has_unfinished():
        engine.step()
        if not cancelled and runner.cache.is_live("r3") and engine._sequences["r3"].status.name == "WAITING":
            engine.cancel("r3")                                            # admitted by the plan ahead, not yet begun
            cancelled = True
            assert not runner.cache.is_live("r3")
        runner.cache.assert_invariants()
    assert cancelled and runner.discarded_ahead >= 2
    assert list(engine.pop_result("r0").token_ids) == expected[0]
    assert list(engine.pop_result("r1").token_ids) == expected[1][:1]
    assert list(engine.pop_result("r2").token_ids) == expected[2]
    assert runner.cache.live_requests() == () and runner.cache.capacity().free_blocks == (64,)
    assert runner.cache.capacity().free_slots == 3

    # requests that arrive while others run, in random order, with few pages: the same tokens
    rng = random.Random(5)
    for trial in range(20):
        engine, runner = make_engine(num_kv_blocks=rng.choice([14, 20, 64]), max_num_seqs=rng.choice([2, 3, 4]), **{
            k: v for k, v in options.items() if k != "max_num_seqs"})
        runner.prepare_ahead = True
        order = list(range(len(PROMPTS)))
        rng.shuffle(order)
        pending = [(rng.randrange(0, 12), index) for index in order]
        step = 0
        while pending or engine.has_unfinished():
            for due, index in list(pending):
                if due <= step:
                    engine.add_request(f"r{index}", PROMPTS[index], params, arrival_ns=step * 10 + index)
                    pending.remove((due, index))
            engine.step()
            runner.cache.assert_invariants()
            step += 1
            assert step < 500
        for index in range(len(PROMPTS)):
            assert list(engine.pop_result(f"r{index}").token_ids) == expected[index], (trial, index)
        assert runner.cache.live_requests() == () and runner.used_ahead > 0


@pytest.mark.parametrize("seed", range(24))
def test_random_serving_never_changes_a_token(seed):
    """Requests of random lengths arrive at random steps, some with stop tokens, some
    cancelled on the way, on pools from roomy to so tight that requests are preempted,
    with prompts whole or in portions, steps planned ahead or not and launched ahead or
    not: every request that ends has generated exactly what its tokens determine, a
    cancelled one a prefix of it; no page or slot is lost at any step or at the end."""

    rng = random.Random(1000 + seed)
    vocab = 97
    blocks = rng.choice([12, 16, 24, 64])
    options = dict(num_kv_blocks=blocks, max_num_seqs=rng.choice([2, 3, 4]))
    if rng.random() < 0.6:
        options.update(enable_chunked_prefill=True, prefill_chunk_size=rng.choice([3, 7, 16]),
                       max_num_batched_tokens=rng.choice([8, 16, 48]))
    engine, runner = make_engine(**options)
    runner.prepare_ahead = rng.random() < 0.7
    if runner.prepare_ahead and rng.random() < 0.7:
        runner.chain = True
        engine.sampler = ArgmaxSampler(on_device=True)
    requests = {}
    for index in range(rng.randrange(3, 9)):
        # (a request never needs more pages than the pool has: 4 tokens a page)
        prompt = [rng.randrange(vocab) for _ in range(rng.randrange(1, min(40, 4 * blocks - 24)))]
        new_tokens = rng.randrange(1, 21)
        whole = expected_generation(prompt, new_tokens, vocab)
        stops = (whole[rng.randrange(len(whole))],) if rng.random() < 0.3 else ()
        requests[f"r{index}"] = dict(
            prompt=prompt, params=SamplingParams(max_new_tokens=new_tokens, stop_token_ids=stops),
            expected=expected_generation(prompt, new_tokens, vocab, stop=stops), due=rng.randrange(0, 25),
            cancel_at=rng.randrange(1, 40) if rng.random() < 0.2 else None)
    pending = dict(requests)
    cancelled = set()
    step = 0
    while pending or engine.has_unfinished():
        for name, request in list(pending.items()):
            if request["due"] <= step:
                engine.add_request(name, request["prompt"], request["params"], arrival_ns=step * 100 + int(name[1:]))
                del pending[name]
        for name, request in requests.items():
            if request["cancel_at"] == step and name in engine._sequences:
                engine.cancel(name)
                cancelled.add(name)
        if engine.has_unfinished():
            engine.step()
        runner.cache.assert_invariants()
        step += 1
        assert step < 2000
    for name, request in requests.items():
        result = engine.pop_result(name)
        got = list(result.token_ids)
        if name in cancelled:
            assert got == request["expected"][: len(got)] and len(got) < len(request["expected"])
        else:
            assert got == request["expected"], (name, result.finish_reason)
            assert result.finish_reason == ("stop" if got[-1] in request["params"].stop_token_ids else "length")
    capacity = runner.cache.capacity()
    assert runner.cache.live_requests() == () and capacity.free_blocks == (blocks,)
    assert capacity.free_slots == options["max_num_seqs"]
    if runner.chain:
        assert runner.chained >= runner.voided_chained


def test_stop_tokens_and_per_request_parameters():
    engine, _ = make_engine()
    first = expected_generation(PROMPTS[0], 12, 97)
    stop = first[3]
    params = [SamplingParams(max_new_tokens=12, stop_token_ids=(stop,)), SamplingParams(max_new_tokens=2)]
    out = engine.generate(PROMPTS[:2], params)
    assert out[0] == first[: first.index(stop) + 1] and out[1] == expected_generation(PROMPTS[1], 2, 97)


def test_admission_checks():
    # reference: miniserve/engine/core.py:193-236
    engine, _ = make_engine(num_kv_blocks=8)
    engine.add_request("a", [1, 2, 3])
    with pytest.raises(ValueError, match="Duplicate"):
        engine.add_request("a", [1])
    with pytest.raises(ValueError, match="CONTEXT_LENGTH_EXCEEDED"):
        engine.add_request("b", [1] * 120, SamplingParams(max_new_tokens=9))
    with pytest.raises(ValueError, match="CONTEXT_CAPACITY_EXCEEDED"):
        engine.add_request("c", [1] * 30, SamplingParams(max_new_tokens=8))
    with pytest.raises(ValueError, match="outside the vocabulary"):
        engine.add_request("d", [97])
    with pytest.raises(ValueError, match="top_k"):
        engine.add_request("e", [1], SamplingParams(temperature=1.0, top_k=98))
    with pytest.raises(ValueError, match="stop token"):
        engine.add_request("f", [1], SamplingParams(stop_token_ids=(500,)))
    small, _ = make_engine(max_num_batched_tokens=16)
    with pytest.raises(ValueError, match="CHUNKED_PREFILL_DISABLED"):
        small.add_request("g", [1] * 20)
    full, _ = make_engine(max_pending_requests=1)
    full.add_request("h", [1])
    with pytest.raises(RuntimeError, match="QUEUE_FULL"):
        full.add_request("i", [1])


def test_a_failed_step_leaves_no_trace_and_fails_its_requests():
    engine, runner = make_engine(fail_on_step=1)
    engine.add_request("a", [1, 2, 3], SamplingParams(max_new_tokens=4), arrival_ns=0)
    engine.step()
    with pytest.raises(RuntimeError, match="injected"):
        engine.step()
    assert engine.pop_result("a").finish_reason == "error"
    assert runner.cache.capacity().free_blocks == (64,) and runner.cache.live_requests() == ()
    engine.add_request("b", [1, 2, 3], SamplingParams(max_new_tokens=4), arrival_ns=1)
    while engine.has_unfinished():
        engine.step()
    assert list(engine.pop_result("b").token_ids) == expected_generation([1, 2, 3], 4, 97)


def test_cancel_gives_everything_back():
    engine, runner = make_engine()
    engine.add_request("a", list(range(9)), SamplingParams(max_new_tokens=5))
    engine.step()
    engine.cancel("a")
    assert runner.cache.capacity().free_blocks == (64,) and not engine.has_unfinished()
    assert engine.pop_result("a").finish_reason == "cancelled"


def test_recorded_context_bounds():
    from miniserve_amd.engine.runner import recorded_context_bound

    assert [recorded_context_bound(n, 40960) for n in (1, 100, 256, 257, 2049, 4096, 33000, 40960)] == [
        256, 256, 256, 512, 4096, 4096, 40960, 40960]
    assert recorded_context_bound(100, 128) == 128
