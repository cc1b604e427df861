"""Continuous batching with chunked prefill under a token budget.

Reference: kvcore/sched/scheduler.py:147-302 (``schedule``: running requests first,
then waiting ones first come first served; a request's share is what it has left,
capped by ``long_prefill_token_threshold`` and by the budget), :418-523 (one request),
:333-416 (``update_from_outputs``: advance, take the sampled token when every known
token is computed, finish on a stop token or the length cap, free) and :541-577 (limits
on requests that are still in their prompt).

When pages run out.  The reference has no preemption: a running request that cannot
grow stops the pass, and if nothing could be scheduled the engine raises
(scheduler.py:195-196,264-273; kvcore/entry/llm_engine.py:66-73).  Here a running
request that cannot get its pages takes them from the running request that was admitted
last (possibly itself): that one gives back all its pages and its slot, returns to the
front of the waiting queue with nothing computed, and later computes prompt and
generated tokens again as one prompt.  Its output so far is kept, so nothing is
sampled twice.  ``add_request`` refuses what could never fit, so the no-progress error
remains only as a guard.
"""

from __future__ import annotations

from collections import deque
from dataclasses import dataclass, field
from typing import Iterable, Mapping

from kvcore_amd.cache.kv_manager import KVManager, cdiv
from kvcore_amd.config.engine_config import SchedulerConfig
from kvcore_amd.sampling.params import SamplingParams

from .request import FinishReason, Request, RequestStatus

AHEAD_TOKEN = -1  # stands for a token that the device holds and the host does not know yet


@dataclass(frozen=True)
class ScheduledRequest:
    """One request's share of a step.  ``is_new`` marks the first step after admission
    (or after a preemption): ``token_ids`` then starts at position 0 of the request.
    The reference sends ``NewRequestData`` / ``CachedRequestData`` (kvcore/sched/
    utils.py:10-75); both carry what this record carries."""

    request_id: str
    slot: int
    is_new: bool
    token_ids: tuple[int, ...]
    num_computed_tokens: int
    page_ids: tuple[tuple[int, ...], ...]
    released: tuple[int, ...]
    samples: bool  # this share reaches the request's last known token
    num_output_tokens: int
    sampling_params: SamplingParams


@dataclass(frozen=True)
class SchedulerOutput:
    scheduled: tuple[ScheduledRequest, ...] = ()
    num_scheduled_tokens: Mapping[str, int] = field(default_factory=dict)
    total_num_scheduled_tokens: int = 0
    finished_req_ids: frozenset[str] = frozenset()
    preempted_req_ids: tuple[str, ...] = ()
    step_id: int = 0

    @property
    def is_empty(self) -> bool:
        return self.total_num_scheduled_tokens == 0


@dataclass(frozen=True)
class RequestStepOutput:
    request_id: str
    sampled_token_id: int | None
    finished: bool
    finish_reason: FinishReason | None


@dataclass(frozen=True)
class FinishedRequestState:
    request_id: str
    output_token_ids: tuple[int, ...]
    finish_reason: FinishReason | None


@dataclass(frozen=True)
class SchedulerUpdateResult:
    step_outputs: tuple[RequestStepOutput, ...] = ()
    finished_requests: tuple[FinishedRequestState, ...] = ()


@dataclass(frozen=True)
class SchedulerNoProgressState:
    waiting: tuple[str, ...]
    running: tuple[str, ...]
    free_pages: tuple[int, ...]
    max_num_seqs: int
    max_num_scheduled_tokens: int

    def format_message(self) -> str:
        return (
            "Scheduler made no progress "
            f"(waiting={self.waiting}, running={self.running}, free_pages={self.free_pages}, "
            f"max_num_seqs={self.max_num_seqs}, "
            f"max_num_scheduled_tokens={self.max_num_scheduled_tokens})"
        )


class Scheduler:
    def __init__(self, config: SchedulerConfig, kv_manager: KVManager, *, max_model_len: int) -> None:
        self.config = config
        self.kv_manager = kv_manager
        self.max_model_len = max_model_len
        self.requests: dict[str, Request] = {}
        self.waiting: deque[Request] = deque()
        self.running: list[Request] = []
        self.finished_req_ids: set[str] = set()
        self.last_no_progress_state: SchedulerNoProgressState | None = None
        self.step_id = 0
        self.num_preemptions = 0

    # ---------------------------------------------------------------------- admission
    def add_request(self, request: Request) -> None:
        """Queue a request.  Refuses a duplicate id (scheduler.py:83-85) and, beyond the
        reference, a request that could never finish: longer than ``max_model_len`` or
        than the whole page pool."""
        if request.request_id in self.requests:
            raise ValueError(f"Duplicate request_id: {request.request_id}")
        total = request.num_prompt_tokens + request.max_tokens
        if total > self.max_model_len:
            raise ValueError(
                f"request {request.request_id!r}: prompt ({request.num_prompt_tokens}) plus max_tokens "
                f"({request.max_tokens}) exceeds max_model_len={self.max_model_len}")
        for group, pool in zip(self.kv_manager.groups, self.kv_manager.pools):
            need = cdiv(total, group.page_size)
            if group.window > 0:
                need = min(need, cdiv(group.window + self.config.max_num_scheduled_tokens, group.page_size) + 1)
            if need > pool.num_usable:
                raise ValueError(
                    f"request {request.request_id!r} needs {need} cache pages of {group.page_size} "
                    f"tokens; the pool has {pool.num_usable}")
        self.requests[request.request_id] = request
        self.waiting.append(request)

    def get_num_unfinished_requests(self) -> int:
        return len(self.running) + len(self.waiting)

    def has_unfinished_requests(self) -> bool:
        return bool(self.running or self.waiting)

    def get_request_counts(self) -> tuple[int, int]:
        return len(self.running), len(self.waiting)

    # ------------------------------------------------------------------------ helpers
    def _is_prefill(self, request: Request) -> bool:
        """Still in its prompt (scheduler.py:541-543), where "prompt" includes, after a
        preemption, the output that is computed again with it."""
        return request.num_computed_tokens < request.num_prefill_tokens

    def _is_long_prefill(self, request: Request) -> bool:
        threshold = self.config.long_prefill_token_threshold
        return threshold > 0 and request.num_prefill_tokens >= threshold

    def _can_schedule_partial_prefill(self, request: Request, num_partial: int, num_long: int) -> bool:
        if num_partial >= self.config.max_num_partial_prefills:
            return False
        return not (self._is_long_prefill(request) and num_long >= self.config.max_long_partial_prefills)

    def _share(self, request: Request, budget: int) -> int:
        remaining = request.num_tokens - request.num_computed_tokens
        threshold = self.config.long_prefill_token_threshold
        if 0 < threshold < remaining:
            remaining = threshold
        return min(remaining, budget)

    def _preempt(self, request: Request) -> None:
        self.kv_manager.free(request.request_id)
        request.status = RequestStatus.PREEMPTED
        request.num_computed_tokens = 0
        request.num_prefill_tokens = request.num_tokens  # all of it is a prompt now
        request.num_preemptions += 1
        self.num_preemptions += 1
        self.running.remove(request)
        self.waiting.appendleft(request)

    def _emit(self, request: Request, n: int, is_new: bool) -> ScheduledRequest:
        start = request.num_computed_tokens
        rid = request.request_id
        return ScheduledRequest(
            request_id=rid,
            slot=self.kv_manager.slot_of(rid),
            is_new=is_new,
            token_ids=tuple(request.all_token_ids[start:start + n]),
            num_computed_tokens=start,
            page_ids=tuple(tuple(p) for p in self.kv_manager.page_ids(rid)),
            released=tuple(self.kv_manager.released_counts(rid)),
            samples=start + n >= request.num_tokens,
            num_output_tokens=request.num_output_tokens,
            sampling_params=request.sampling_params,
        )

    # ----------------------------------------------------------------------- schedule
    def schedule(self) -> SchedulerOutput:
        self.last_no_progress_state = None
        budget = self.config.max_num_scheduled_tokens
        max_num_seqs = self.config.max_num_seqs
        scheduled: list[ScheduledRequest] = []
        num_scheduled: dict[str, int] = {}
        preempted: list[str] = []
        num_partial = num_long = 0

        # pass 1: running requests, in the order they were admitted
        index = 0
        while index < len(self.running) and len(num_scheduled) < max_num_seqs and budget > 0:
            request = self.running[index]
            is_prefill = self._is_prefill(request)
            if is_prefill and not self._can_schedule_partial_prefill(request, num_partial, num_long):
                break
            n = self._share(request, budget)
            if n <= 0:
                break
            got = self.kv_manager.allocate(request.request_id, request.num_computed_tokens, n)
            while got is None:
                victim = self.running[-1]
                if victim.request_id in num_scheduled:
                    break  # everything behind is already part of this step
                self._preempt(victim)
                preempted.append(victim.request_id)
                if victim is request:
                    break
                got = self.kv_manager.allocate(request.request_id, request.num_computed_tokens, n)
            if got is None:
                break
            scheduled.append(self._emit(request, n, is_new=False))
            num_scheduled[request.request_id] = n
            if is_prefill:
                num_partial += 1
                num_long += self._is_long_prefill(request)
            budget -= n
            index += 1

        # pass 2: waiting requests, first come first served
        skipped: list[Request] = []
        while self.waiting and not preempted and len(num_scheduled) < max_num_seqs and budget > 0:
            request = self.waiting[0]
            if not self.kv_manager.has_free_slot():
                break
            if not self._can_schedule_partial_prefill(request, num_partial, num_long):
                skipped.append(self.waiting.popleft())  # set aside, keep scanning (scheduler.py:235-242)
                continue
            n = self._share(request, budget)
            if n <= 0 or not self.kv_manager.can_fit(request.request_id, request.num_computed_tokens + n):
                break
            self.waiting.popleft()
            self.kv_manager.admit(request.request_id)
            got = self.kv_manager.allocate(request.request_id, request.num_computed_tokens, n)
            assert got is not None
            request.status = RequestStatus.RUNNING
            self.running.append(request)
            scheduled.append(self._emit(request, n, is_new=True))
            num_scheduled[request.request_id] = n
            num_partial += 1
            num_long += self._is_long_prefill(request)
            budget -= n
        for request in reversed(skipped):
            self.waiting.appendleft(request)

        finished = frozenset(self.finished_req_ids)
        self.finished_req_ids.clear()
        total = sum(num_scheduled.values())
        if total == 0 and not finished and not preempted:
            self.last_no_progress_state = SchedulerNoProgressState(
                waiting=tuple(r.request_id for r in self.waiting),
                running=tuple(r.request_id for r in self.running),
                free_pages=tuple(self.kv_manager.num_free_pages()),
                max_num_seqs=max_num_seqs,
                max_num_scheduled_tokens=self.config.max_num_scheduled_tokens,
            )
            return SchedulerOutput(step_id=self.step_id)
        return SchedulerOutput(tuple(scheduled), num_scheduled, total, finished, tuple(preempted),
                               self.step_id)

    # --------------------------------------------------------------------- run ahead
    def plan_decode_ahead(self, output: SchedulerOutput) -> SchedulerOutput | None:
        """The step that follows ``output`` if no request of ``output`` ends on a stop token,
        made before ``output``'s sampled tokens are known: the same requests in the same
        order, one position further, the token itself being ``AHEAD_TOKEN`` (the caller
        takes it from where the device left the sampled one).  Only a step of single
        decoded tokens that holds every running request is continued, and only if nothing
        waits that a free slot could take, no request reaches its length cap or the context
        limit with ``output``, and every page the next position needs is free: in every
        other case the answer is None and the caller goes the ordinary way (``update`` then
        ``schedule``), which decides what this method does not.  Pages are taken at once;
        a request that ends after all gives them back with the rest of its pages.  A cache
        group with a window gives back, also at once, the pages that ``output`` moves the
        window past, in the order in which ``update_from_outputs`` would (all requests first,
        then the new pages are taken): ``output`` has been launched, the planned step follows it
        on the same stream, so whoever gets such a page writes it after ``output`` has read it.
        The requests themselves are not touched: ``update_from_outputs`` takes the planned
        step as it takes any other, once it has taken ``output``."""
        if not output.scheduled or output.preempted_req_ids:
            return None
        if self.waiting and self.kv_manager.has_free_slot():
            return None  # with every slot taken nobody can be admitted (``schedule``, pass 2)
        if len(output.scheduled) != len(self.running):
            return None
        for s, request in zip(output.scheduled, self.running):
            if s.request_id != request.request_id or len(s.token_ids) != 1 or not s.samples or s.is_new:
                return None
            if s.num_output_tokens + 1 >= request.max_tokens:
                return None  # ends with ``output``
            if s.num_computed_tokens + 2 > self.max_model_len:
                return None
        if any(g.window > 0 for g in self.kv_manager.groups):
            for s in output.scheduled:  # what ``update_from_outputs`` will find done already
                self.kv_manager.release_behind_window(s.request_id, s.num_computed_tokens + 1)
        planned: list[ScheduledRequest] = []
        for s in output.scheduled:
            start = s.num_computed_tokens + 1
            if self.kv_manager.allocate(s.request_id, start, 1) is None:
                return None  # pages already taken for others are theirs one step early
            planned.append(ScheduledRequest(
                request_id=s.request_id, slot=s.slot, is_new=False, token_ids=(AHEAD_TOKEN,),
                num_computed_tokens=start,
                page_ids=tuple(tuple(p) for p in self.kv_manager.page_ids(s.request_id)),
                released=tuple(self.kv_manager.released_counts(s.request_id)), samples=True,
                num_output_tokens=s.num_output_tokens + 1, sampling_params=s.sampling_params))
        return SchedulerOutput(tuple(planned), {s.request_id: 1 for s in planned}, len(planned),
                               frozenset(), (), output.step_id + 1)

    def without_finished(self, output: SchedulerOutput) -> SchedulerOutput:
        """``output`` without the requests that have ended since it was planned."""
        alive = tuple(s for s in output.scheduled if s.request_id in self.requests)
        if len(alive) == len(output.scheduled):
            return output
        return SchedulerOutput(alive, {s.request_id: len(s.token_ids) for s in alive},
                               sum(len(s.token_ids) for s in alive), output.finished_req_ids,
                               output.preempted_req_ids, output.step_id)

    # ------------------------------------------------------------------------- update
    def update_from_outputs(self, output: SchedulerOutput, sampled_token_ids: Mapping[str, int], *,
                            stop_token_ids: Iterable[int] | None = None) -> SchedulerUpdateResult:
        stop = set(stop_token_ids or ())
        step_outputs: list[RequestStepOutput] = []
        finished_requests: list[FinishedRequestState] = []
        for request_id, n in output.num_scheduled_tokens.items():
            request = self.requests[request_id]
            request.num_computed_tokens += n
            sampled: int | None = None
            finished = False
            reason: FinishReason | None = None
            if request.num_computed_tokens >= request.num_tokens:
                sampled = int(sampled_token_ids[request_id])
                request.append_output_token(sampled)
                if sampled in stop and not request.sampling_params.ignore_eos:
                    request.status = RequestStatus.FINISHED_STOPPED
                elif request.num_output_tokens >= request.max_tokens:
                    request.status = RequestStatus.FINISHED_LENGTH_CAPPED
                if request.is_finished():
                    finished = True
                    reason = request.finish_reason()
                    finished_requests.append(self._free_finished(request))
            if not finished:
                self.kv_manager.release_behind_window(request_id, request.num_computed_tokens)
            step_outputs.append(RequestStepOutput(request_id, sampled, finished, reason))
        self.step_id += 1
        return SchedulerUpdateResult(tuple(step_outputs), tuple(finished_requests))

    def _free_finished(self, request: Request) -> FinishedRequestState:
        if self.kv_manager.is_admitted(request.request_id):
            self.kv_manager.free(request.request_id)
        if request in self.running:
            self.running.remove(request)
        self.requests.pop(request.request_id, None)
        self.finished_req_ids.add(request.request_id)
        return FinishedRequestState(request.request_id, tuple(request.output_token_ids),
                                    request.finish_reason())

    def finish_requests(self, request_ids: str | Iterable[str] | None,
                        finished_status: RequestStatus) -> tuple[FinishedRequestState, ...]:
        """Abort (or otherwise end) requests wherever they are (scheduler.py:98-133)."""
        if not RequestStatus.is_finished(finished_status):
            raise ValueError(f"finished_status must be a finished status, got {finished_status}")
        if isinstance(request_ids, str):
            ids = {request_ids}
        elif request_ids is None:
            ids = set(self.requests)
        else:
            ids = set(request_ids)
        out = []
        for rid in ids:
            request = self.requests.get(rid)
            if request is None or request.is_finished():
                continue
            request.status = finished_status
            if request in self.waiting:
                self.waiting.remove(request)
            out.append(self._free_finished(request))
        return tuple(out)

    def shutdown(self) -> None:
        self.finish_requests(None, RequestStatus.FINISHED_ABORTED)
