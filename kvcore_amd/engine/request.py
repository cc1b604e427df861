"""A request's state as the scheduler sees it.

Reference: kvcore/utils/request.py:13-46 (finish reasons and statuses; finished means
greater than PREEMPTED) and :78-160 (token lists and counters).  Streaming, priority,
event and prefix-hash fields have no counterpart here.
"""

from __future__ import annotations

import enum
from typing import Sequence

from kvcore_amd.sampling.params import SamplingParams


class FinishReason(enum.Enum):
    STOP = "stop"
    LENGTH = "length"
    ABORT = "abort"
    ERROR = "error"


class RequestStatus(enum.IntEnum):
    WAITING = enum.auto()
    RUNNING = enum.auto()
    PREEMPTED = enum.auto()
    FINISHED_STOPPED = enum.auto()
    FINISHED_LENGTH_CAPPED = enum.auto()
    FINISHED_ABORTED = enum.auto()
    FINISHED_ERROR = enum.auto()

    @staticmethod
    def is_finished(status: "RequestStatus") -> bool:
        return status > RequestStatus.PREEMPTED


_FINISH_REASON = {
    RequestStatus.FINISHED_STOPPED: FinishReason.STOP,
    RequestStatus.FINISHED_LENGTH_CAPPED: FinishReason.LENGTH,
    RequestStatus.FINISHED_ABORTED: FinishReason.ABORT,
    RequestStatus.FINISHED_ERROR: FinishReason.ERROR,
}


class Request:
    def __init__(self, request_id: str, prompt_token_ids: Sequence[int],
                 sampling_params: SamplingParams) -> None:
        if len(prompt_token_ids) == 0:
            raise ValueError("prompt_token_ids must not be empty")  # request.py:93-94
        self.request_id = request_id
        self.prompt_token_ids = list(prompt_token_ids)
        self.sampling_params = sampling_params
        self.max_tokens = sampling_params.max_tokens
        self.output_token_ids: list[int] = []
        self.all_token_ids: list[int] = list(prompt_token_ids)
        self.num_computed_tokens = 0
        self.status = RequestStatus.WAITING
        self.num_preemptions = 0
        # how many leading tokens count as "prompt" for the scheduler's limits on requests
        # that are still prefilling: the prompt, or, after a preemption, the prompt and the
        # output so far, which are computed again as one prompt
        self.num_prefill_tokens = len(self.prompt_token_ids)

    @property
    def num_prompt_tokens(self) -> int:
        return len(self.prompt_token_ids)

    @property
    def num_tokens(self) -> int:
        return len(self.all_token_ids)

    @property
    def num_output_tokens(self) -> int:
        return len(self.output_token_ids)

    def append_output_token(self, token_id: int) -> None:
        self.output_token_ids.append(token_id)
        self.all_token_ids.append(token_id)

    def is_finished(self) -> bool:
        return RequestStatus.is_finished(self.status)

    def finish_reason(self) -> FinishReason | None:
        return _FINISH_REASON.get(self.status)
