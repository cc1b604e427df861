"""The scheduler's decisions, driven without a GPU: a fake step just names tokens."""

from __future__ import annotations

import random

import pytest

from kvcore_amd.cache.kv_manager import GroupConfig, KVManager
from kvcore_amd.config.engine_config import SchedulerConfig
from kvcore_amd.engine.request import FinishReason, Request, RequestStatus
from kvcore_amd.engine.scheduler import Scheduler
from kvcore_amd.sampling.params import SamplingParams


def make_scheduler(config=None, *, num_pages=16, page=2, max_len=16, window=0):
    config = config or SchedulerConfig()
    manager = KVManager([GroupConfig(page, num_pages, window)], max_num_seqs=config.max_num_seqs,
                        max_model_len=max_len)
    return Scheduler(config, manager, max_model_len=max_len)


def make_request(rid, prompt, max_tokens, **kw):
    return Request(rid, prompt, SamplingParams(max_tokens=max_tokens, temperature=0.0, **kw))


def shares(output):
    return {s.request_id: s for s in output.scheduled}


def test_chunked_prefill_continuation_samples_on_the_last_chunk():
    """tests/test_scheduler.py:91-114: 6 tokens under a budget of 4 -> 4, then 2, then the
    sampled token alone."""
    s = make_scheduler(SchedulerConfig(max_num_seqs=1, max_num_scheduled_tokens=4))
    s.add_request(make_request("req", [1, 2, 3, 4, 5, 6], max_tokens=2))
    first = s.schedule()
    assert first.num_scheduled_tokens == {"req": 4} and first.total_num_scheduled_tokens == 4
    share = shares(first)["req"]
    assert share.is_new and share.token_ids == (1, 2, 3, 4) and share.num_computed_tokens == 0
    assert not share.samples and share.page_ids == ((1, 2),)
    s.update_from_outputs(first, {})
    second = s.schedule()
    share = shares(second)["req"]
    assert second.num_scheduled_tokens == {"req": 2}
    assert not share.is_new and share.token_ids == (5, 6) and share.num_computed_tokens == 4
    assert share.samples
    s.update_from_outputs(second, {"req": 9})
    third = s.schedule()
    share = shares(third)["req"]
    assert third.num_scheduled_tokens == {"req": 1}
    assert share.token_ids == (9,) and share.num_output_tokens == 1 and share.samples


def test_partial_prefill_limit():
    """tests/test_scheduler.py:117-133: one prefilling request per step by default."""
    s = make_scheduler(SchedulerConfig(max_num_seqs=2, max_num_scheduled_tokens=4, max_num_partial_prefills=1))
    s.add_request(make_request("req-1", [1, 2, 3, 4, 5, 6], max_tokens=1))
    s.add_request(make_request("req-2", [7, 8, 9, 10, 11, 12], max_tokens=1))
    assert tuple(s.schedule().num_scheduled_tokens) == ("req-1",)


def test_long_prefill_threshold_caps_a_share_and_limits_long_requests():
    cfg = SchedulerConfig(max_num_seqs=4, max_num_scheduled_tokens=12, max_num_partial_prefills=4,
                          max_long_partial_prefills=1, long_prefill_token_threshold=3)
    s = make_scheduler(cfg, num_pages=40, max_len=32)
    s.add_request(make_request("long-1", list(range(8)), max_tokens=1))
    s.add_request(make_request("long-2", list(range(8)), max_tokens=1))
    s.add_request(make_request("short", [1, 2], max_tokens=1))
    out = s.schedule()
    # long-1 gets the threshold, long-2 is set aside (one long prefill at a time), short goes
    assert out.num_scheduled_tokens == {"long-1": 3, "short": 2}
    assert [r.request_id for r in s.waiting] == ["long-2"]


def test_running_requests_go_before_waiting_ones():
    """tests/test_scheduler.py:157-177."""
    s = make_scheduler(SchedulerConfig(max_num_seqs=2, max_num_scheduled_tokens=4, max_num_partial_prefills=2))
    s.add_request(make_request("running", [1, 2, 3, 4, 5, 6], max_tokens=1))
    first = s.schedule()
    s.update_from_outputs(first, {})
    s.add_request(make_request("waiting", [7, 8], max_tokens=1))
    second = s.schedule()
    assert tuple(second.num_scheduled_tokens) == ("running", "waiting")
    assert second.num_scheduled_tokens == {"running": 2, "waiting": 2}


def test_decode_progression_and_length_finish():
    """tests/test_scheduler.py:180-198."""
    s = make_scheduler(SchedulerConfig(max_num_seqs=2, max_num_scheduled_tokens=4))
    s.add_request(make_request("req", [1, 2, 3, 4], max_tokens=2))
    first = s.schedule()
    update = s.update_from_outputs(first, {"req": 9})
    assert update.step_outputs[0].sampled_token_id == 9 and not update.step_outputs[0].finished
    second = s.schedule()
    assert second.num_scheduled_tokens == {"req": 1}
    final = s.update_from_outputs(second, {"req": 10})
    assert final.step_outputs[0].finished and final.step_outputs[0].finish_reason == FinishReason.LENGTH
    assert final.finished_requests[0].output_token_ids == (9, 10)
    assert s.kv_manager.num_free_pages() == [15] and not s.has_unfinished_requests()
    assert s.schedule().finished_req_ids == frozenset({"req"})
    assert s.schedule().finished_req_ids == frozenset()


def test_stop_token_is_kept_and_ignore_eos_skips_it():
    s = make_scheduler(SchedulerConfig(max_num_seqs=2, max_num_scheduled_tokens=8, max_num_partial_prefills=2))
    s.add_request(make_request("stops", [1, 2], max_tokens=5))
    s.add_request(make_request("goes-on", [3, 4], max_tokens=5, ignore_eos=True))
    out = s.schedule()
    upd = s.update_from_outputs(out, {"stops": 7, "goes-on": 7}, stop_token_ids={7})
    by_id = {o.request_id: o for o in upd.step_outputs}
    assert by_id["stops"].finished and by_id["stops"].finish_reason == FinishReason.STOP
    assert upd.finished_requests[0].output_token_ids == (7,)  # scheduler.py:381-384 keeps the stop token
    assert not by_id["goes-on"].finished


def test_admission_refuses_what_can_never_fit():
    s = make_scheduler(num_pages=4, page=2, max_len=16)  # 3 usable pages = 6 tokens
    with pytest.raises(ValueError, match="Duplicate"):
        s.add_request(make_request("a", [1], 1))
        s.add_request(make_request("a", [1], 1))
    with pytest.raises(ValueError, match="max_model_len"):
        s.add_request(make_request("b", list(range(10)), 7))
    with pytest.raises(ValueError, match="cache pages"):
        s.add_request(make_request("c", list(range(5)), 2))
    with pytest.raises(ValueError, match="empty"):
        make_request("d", [], 1)


def test_abort_frees_pages_in_mid_prefill():
    s = make_scheduler(SchedulerConfig(max_num_seqs=2, max_num_scheduled_tokens=4))
    s.add_request(make_request("req", list(range(1, 9)), max_tokens=1))
    s.add_request(make_request("queued", [1, 2], max_tokens=1))
    s.update_from_outputs(s.schedule(), {})
    assert s.kv_manager.num_free_pages() == [13]
    done = s.finish_requests(None, RequestStatus.FINISHED_ABORTED)
    assert {d.request_id for d in done} == {"req", "queued"}
    assert all(d.finish_reason == FinishReason.ABORT for d in done)
    assert s.kv_manager.num_free_pages() == [15] and not s.has_unfinished_requests()
    s.kv_manager.check()
    with pytest.raises(ValueError):
        s.finish_requests("x", RequestStatus.RUNNING)


def test_when_pages_run_out_the_last_admitted_request_is_preempted_and_recomputed():
    # 6 usable pages of 2 tokens.  Two requests of 4 prompt tokens take 2 pages each; each decode
    # step needs a page per request every second token, so the pool runs dry.
    cfg = SchedulerConfig(max_num_seqs=2, max_num_scheduled_tokens=8, max_num_partial_prefills=2)
    s = make_scheduler(cfg, num_pages=7, page=2, max_len=12)
    s.add_request(make_request("first", [1, 2, 3, 4], max_tokens=6))
    s.add_request(make_request("second", [5, 6, 7, 8], max_tokens=6))
    token = 100
    preempted_seen = False
    outputs = {"first": [], "second": []}
    for _ in range(60):
        if not s.has_unfinished_requests():
            break
        out = s.schedule()
        assert sum(out.num_scheduled_tokens.values()) <= 8
        if out.preempted_req_ids:
            preempted_seen = True
            assert out.preempted_req_ids == ("second",)  # the one admitted last
            assert s.requests["second"].num_computed_tokens == 0
            assert s.requests["second"].status == RequestStatus.PREEMPTED
            assert s.waiting[0].request_id == "second"
        sampled = {}
        for share in out.scheduled:
            if share.samples:
                token += 1
                sampled[share.request_id] = token
                outputs[share.request_id].append(token)
            if share.is_new and s.requests[share.request_id].num_preemptions:
                # recomputation: prompt and generated tokens again as one prompt
                assert share.num_computed_tokens == 0
                assert share.token_ids[:4] == (5, 6, 7, 8) and len(share.token_ids) > 4
        s.update_from_outputs(out, sampled)
        s.kv_manager.check()
    assert preempted_seen and s.num_preemptions >= 1
    assert not s.has_unfinished_requests()
    assert len(outputs["first"]) == 6 and len(outputs["second"]) == 6  # nothing sampled twice
    assert s.kv_manager.num_free_pages() == [6]


def test_a_request_that_recomputes_after_preemption_counts_as_a_prefill():
    """After a preemption the prompt and the output so far are computed again as one prompt;
    while that lasts the request counts against ``max_num_partial_prefills`` (and, by its new
    length, against the limit on long ones), also beyond its original prompt's length."""
    cfg = SchedulerConfig(max_num_seqs=3, max_num_scheduled_tokens=3, max_num_partial_prefills=1,
                          long_prefill_token_threshold=0)
    s = make_scheduler(cfg, num_pages=40, page=2, max_len=32)
    victim = make_request("victim", [1, 2], max_tokens=12)
    s.add_request(victim)
    for token in range(6):  # prompt, then five decode steps: 2 + 6 tokens known
        out = s.schedule()
        s.update_from_outputs(out, {"victim": 50 + token})
    assert victim.num_tokens == 8 and not s._is_prefill(victim)
    s._preempt(victim)
    assert victim.num_prefill_tokens == 8 and s._is_prefill(victim)
    s.add_request(make_request("other", [7, 8, 9, 10], max_tokens=2))
    out = s.schedule()  # budget 3: the victim recomputes tokens 0..2 and is the one prefill
    assert out.num_scheduled_tokens == {"victim": 3}
    s.update_from_outputs(out, {})
    out = s.schedule()  # past its prompt's two tokens, it is still the one prefill allowed
    assert victim.num_computed_tokens == 3 and s._is_prefill(victim)
    assert out.num_scheduled_tokens == {"victim": 3}
    s.update_from_outputs(out, {})
    out = s.schedule()
    assert out.num_scheduled_tokens == {"victim": 2} and shares(out)["victim"].samples
    s.update_from_outputs(out, {"victim": 99})
    assert not s._is_prefill(victim)
    out = s.schedule()  # now it decodes, and the other request may start its prompt
    assert out.num_scheduled_tokens == {"victim": 1, "other": 2}
    # a long recomputation is a long prefill
    cfg = SchedulerConfig(max_num_seqs=3, max_num_scheduled_tokens=16, max_num_partial_prefills=3,
                          max_long_partial_prefills=1, long_prefill_token_threshold=4)
    s = make_scheduler(cfg, num_pages=40, page=2, max_len=32)
    victim = make_request("victim", [1, 2], max_tokens=12)
    s.add_request(victim)
    for token in range(5):
        s.update_from_outputs(s.schedule(), {"victim": 50 + token})
    assert not s._is_long_prefill(victim)
    s._preempt(victim)
    assert s._is_long_prefill(victim)
    s.add_request(make_request("long", list(range(6)), max_tokens=1))
    out = s.schedule()
    assert out.num_scheduled_tokens == {"victim": 4}  # one long prefill at a time


def test_no_progress_is_reported_when_nothing_can_run():
    cfg = SchedulerConfig(max_num_seqs=1, max_num_scheduled_tokens=4)
    s = make_scheduler(cfg, num_pages=4, page=2, max_len=6)
    s.add_request(make_request("a", [1, 2, 3], max_tokens=1))
    # someone else holds every page: the waiting request cannot start
    s.kv_manager.admit("squatter")
    s.kv_manager.allocate("squatter", 0, 6)
    out = s.schedule()
    assert out.is_empty and s.last_no_progress_state is not None
    msg = s.last_no_progress_state.format_message()
    assert "waiting=('a',)" in msg and "free_pages=(0,)" in msg


@pytest.mark.parametrize("seed", range(4))
def test_random_traffic_keeps_the_invariants(seed):
    rng = random.Random(seed)
    cfg = SchedulerConfig(max_num_seqs=4, max_num_scheduled_tokens=rng.choice([5, 16]),
                          max_num_partial_prefills=rng.choice([1, 4]), max_long_partial_prefills=2,
                          long_prefill_token_threshold=rng.choice([0, 6]))
    s = make_scheduler(cfg, num_pages=rng.choice([14, 40]), page=4, max_len=48)
    expected = {}
    for i in range(12):
        n_prompt, n_new = rng.randint(1, 30), rng.randint(1, 12)
        s.add_request(make_request(f"r{i}", [rng.randrange(50) for _ in range(n_prompt)], n_new))
        expected[f"r{i}"] = n_new
    finished = {}
    steps = 0
    while s.has_unfinished_requests():
        steps += 1
        assert steps < 2000
        out = s.schedule()
        assert not (out.is_empty and not out.preempted_req_ids and not out.finished_req_ids), \
            s.last_no_progress_state
        assert out.total_num_scheduled_tokens <= cfg.max_num_scheduled_tokens
        assert len(out.scheduled) <= cfg.max_num_seqs
        assert len({sh.slot for sh in out.scheduled}) == len(out.scheduled)
        sampled = {}
        for sh in out.scheduled:
            req = s.requests[sh.request_id]
            assert sh.token_ids == tuple(req.all_token_ids[sh.num_computed_tokens:
                                                           sh.num_computed_tokens + len(sh.token_ids)])
            assert sum(len(p) for p in sh.page_ids) * 4 >= sh.num_computed_tokens + len(sh.token_ids)
            assert sh.samples == (sh.num_computed_tokens + len(sh.token_ids) == req.num_tokens)
            if sh.samples:
                sampled[sh.request_id] = rng.randrange(50)
        upd = s.update_from_outputs(out, sampled)
        for f in upd.finished_requests:
            finished[f.request_id] = f
        s.kv_manager.check()
    assert {k: len(v.output_token_ids) for k, v in finished.items()} == expected
    assert s.kv_manager.num_free_pages() == [s.kv_manager.pools[0].num_usable]
    assert s.kv_manager.slots.num_free == 4


# ------------------------------------------------------------------------ running ahead
def _fake_token(rid, index, stop_at):
    """A request's ``index``-th output: a function of the request and the index alone, as the
    engine's tokens are; request ``rid`` says the stop token 99 at index ``stop_at[rid]``."""
    return 99 if stop_at.get(rid) == index else 100 + (hash((rid, index)) % 50)


def _drive(scheduler, *, ahead, stop_at, arrivals=()):
    """The engine's loop without a device: with ``ahead`` the step after the one whose tokens
    are awaited is planned first, as ``EngineCore.step`` does.  Returns each request's output
    and the requests of every step that ran."""
    outputs, steps = {}, []
    stats = {"planned": 0, "dropped": 0}
    arrivals = dict(arrivals)
    in_flight = None
    for tick in range(400):
        for request in arrivals.pop(tick, ()):
            scheduler.add_request(request)
        if not scheduler.has_unfinished_requests():
            if not arrivals:
                break
            continue
        out, in_flight = in_flight, None
        if out is None:
            out = scheduler.schedule()
            if out.is_empty:
                continue
        steps.append(tuple((s.request_id, s.num_computed_tokens, len(s.token_ids)) for s in out.scheduled))
        planned = scheduler.plan_decode_ahead(out) if ahead else None
        sampled = {s.request_id: _fake_token(s.request_id, s.num_output_tokens, stop_at)
                   for s in out.scheduled if s.samples}
        result = scheduler.update_from_outputs(out, sampled, stop_token_ids={99})
        for state in result.finished_requests:
            outputs[state.request_id] = (state.output_token_ids, state.finish_reason)
        if planned is not None:
            stats["planned"] += 1
            kept = scheduler.without_finished(planned)
            stats["dropped"] += len(planned.scheduled) - len(kept.scheduled)
            in_flight = None if kept.is_empty else kept
    assert not scheduler.has_unfinished_requests()
    return outputs, steps, stats


def test_a_step_planned_ahead_is_the_step_that_would_have_been_scheduled():
    s = make_scheduler(SchedulerConfig(max_num_seqs=4, max_num_scheduled_tokens=16, max_num_partial_prefills=4),
                       num_pages=32, page=2, max_len=24)
    s.add_request(make_request("a", [1, 2, 3], max_tokens=6))
    s.add_request(make_request("b", [4, 5, 6, 7], max_tokens=6))
    first = s.schedule()
    assert s.plan_decode_ahead(first) is None  # prompts: not a step of single decoded tokens
    s.update_from_outputs(first, {"a": 10, "b": 11})
    second = s.schedule()
    planned = s.plan_decode_ahead(second)
    assert planned is not None and planned.step_id == second.step_id + 1
    s.update_from_outputs(second, {"a": 12, "b": 13})
    # what the ordinary way would schedule now, the tokens aside, is what was planned
    pages = {r.request_id: s.kv_manager.page_ids(r.request_id) for r in s.running}
    for share, request in zip(planned.scheduled, s.running):
        assert share.request_id == request.request_id
        assert share.num_computed_tokens == request.num_computed_tokens
        assert share.token_ids == (-1,) and share.samples and not share.is_new
        assert share.num_output_tokens == request.num_output_tokens
        assert [list(p) for p in share.page_ids] == [list(p) for p in pages[request.request_id]]
        assert len(share.page_ids[0]) * 2 > share.num_computed_tokens
    s.update_from_outputs(planned, {"a": 14, "b": 15})
    assert s.requests["a"].output_token_ids[-3:] == [10, 12, 14]


@pytest.mark.parametrize("window", [0, 3, 4])
def test_steps_planned_ahead_with_a_window_are_the_ordinary_steps(window):
    """Two schedulers with the same requests, one planning ahead, one going the ordinary way:
    step for step the same positions, the same page lists (pages that the window has passed
    are given back and read 0) and the same counts of released entries, so the pools hand out
    the same pages in the same order."""
    config = SchedulerConfig(max_num_seqs=3, max_num_scheduled_tokens=16, max_num_partial_prefills=3)
    # with a window a dozen pages serve for good; without one every token keeps its place
    num_pages = 12 if window else 40
    ahead = make_scheduler(config, num_pages=num_pages, page=2, max_len=40, window=window)
    plain_way = make_scheduler(config, num_pages=num_pages, page=2, max_len=40, window=window)
    for sch in (ahead, plain_way):
        sch.add_request(make_request("a", [1, 2, 3, 4, 5], max_tokens=14))
        sch.add_request(make_request("b", [6, 7], max_tokens=14))
        sch.add_request(make_request("c", [8, 9, 10, 11, 12, 13, 14], max_tokens=14))
        sch.update_from_outputs(sch.schedule(), {"a": 20, "b": 21, "c": 22})
    out_a = ahead.schedule()
    planned_steps = 0
    for step in range(12):
        out_b = plain_way.schedule()
        assert [(x.request_id, x.num_computed_tokens, x.page_ids, x.released, x.num_output_tokens)
                for x in out_a.scheduled] == \
               [(x.request_id, x.num_computed_tokens, x.page_ids, x.released, x.num_output_tokens)
                for x in out_b.scheduled], step
        planned = ahead.plan_decode_ahead(out_a)
        tokens = {rid: 30 + step for rid in "abc"}
        ahead.update_from_outputs(out_a, tokens)
        plain_way.update_from_outputs(out_b, tokens)
        ahead.kv_manager.check()
        assert ahead.kv_manager.num_free_pages() == plain_way.kv_manager.num_free_pages() or planned is not None
        if planned is not None:
            planned_steps += 1
            out_a = planned
        else:
            out_a = ahead.schedule()
    assert planned_steps >= 10
    if window:
        assert any(n > 0 for x in out_a.scheduled for n in x.released)  # the window did pass pages
        assert any(0 in pages for x in out_a.scheduled for pages in x.page_ids)


def test_nothing_is_planned_ahead_when_the_ordinary_way_has_something_to_decide():
    config = SchedulerConfig(max_num_seqs=4, max_num_scheduled_tokens=16, max_num_partial_prefills=4)
    # a request reaches its length cap with the step
    s = make_scheduler(config, num_pages=32, max_len=24)
    s.add_request(make_request("a", [1, 2, 3], max_tokens=2))
    s.update_from_outputs(s.schedule(), {"a": 10})
    assert s.plan_decode_ahead(s.schedule()) is None
    # another request waits and a slot is free for it
    s = make_scheduler(config, num_pages=32, max_len=24)
    s.add_request(make_request("a", [1, 2, 3], max_tokens=8))
    s.update_from_outputs(s.schedule(), {"a": 10})
    out = s.schedule()
    s.add_request(make_request("b", [1], max_tokens=2))
    assert s.plan_decode_ahead(out) is None
    # ... but with every slot taken the waiting request changes nothing
    one = SchedulerConfig(max_num_seqs=1, max_num_scheduled_tokens=16)
    s = make_scheduler(one, num_pages=32, max_len=24)
    s.add_request(make_request("a", [1, 2, 3], max_tokens=8))
    s.update_from_outputs(s.schedule(), {"a": 10})
    out = s.schedule()
    s.add_request(make_request("b", [1], max_tokens=2))
    assert s.plan_decode_ahead(out) is not None
    # no page is free for the next position
    s = make_scheduler(config, num_pages=4, page=2, max_len=6)
    s.add_request(make_request("a", [1, 2, 3], max_tokens=3))
    s.add_request(make_request("b", [4], max_tokens=2))
    s.update_from_outputs(s.schedule(), {"a": 10, "b": 11})
    out = s.schedule()  # a: position 3 (page 2 of 2), b: position 1; three pages are out
    assert s.kv_manager.num_free_pages() == [0] and s.plan_decode_ahead(out) is None
    # the context limit
    s = make_scheduler(config, num_pages=32, max_len=5)
    s.add_request(make_request("a", [1, 2, 3], max_tokens=2))
    s.update_from_outputs(s.schedule(), {"a": 10})
    assert s.plan_decode_ahead(s.schedule()) is None


@pytest.mark.parametrize("window", [0, 5])
@pytest.mark.parametrize("seed", range(6))
def test_running_ahead_gives_the_outputs_of_the_ordinary_way(seed, window):
    """Stop tokens at random places (a request that stops has been planned one step too far),
    length caps, arrivals while others decode, and a pool small enough to preempt."""
    rng = random.Random(seed)
    specs, stop_at, arrivals = [], {}, {}
    for i in range(7):
        rid = f"r{i}"
        specs.append((rid, [rng.randrange(50) for _ in range(rng.randint(1, 9))], rng.randint(1, 12)))
        if rng.random() < 0.6:
            stop_at[rid] = rng.randint(0, 8)
        arrivals.setdefault(0 if i < 3 else rng.randint(1, 25), []).append(i)
    results = []
    for ahead in (False, True):
        s = make_scheduler(SchedulerConfig(max_num_seqs=4, max_num_scheduled_tokens=8, max_num_partial_prefills=2),
                           num_pages=rng.choice([14, 40]) if not results else results[0][2], page=2, max_len=24,
                           window=window)
        pool = s.kv_manager.pools[0].num_usable + 1
        arriving = {t: [make_request(*specs[i]) for i in ids] for t, ids in arrivals.items()}
        outputs, steps, stats = _drive(s, ahead=ahead, stop_at=stop_at, arrivals=arriving)
        assert s.kv_manager.num_free_pages() == [s.kv_manager.pools[0].num_usable]
        results.append((outputs, steps, pool, stats))
    assert results[0][0] == results[1][0]
    assert results[1][3]["planned"] > 0
    print("planned ahead", results[1][3], "of", len(results[1][1]), "steps")
    assert set(results[0][0]) == {rid for rid, _, _ in specs}
    for rid, (tokens, reason) in results[1][0].items():
        if rid in stop_at and stop_at[rid] < len(tokens):
            assert tokens[-1] == 99 and reason == FinishReason.STOP
