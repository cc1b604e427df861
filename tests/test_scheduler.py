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
