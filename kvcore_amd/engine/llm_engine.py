"""The Python entry point for offline batches.

Reference: kvcore/entry/llm_engine.py:15-107 (``GenerationRequest``,
``GenerationOutput``, ``add_request``, ``step``, ``generate`` with its no-progress
error).  A request may carry ``prompt_token_ids`` instead of ``messages``; a folder of
random weights has no tokenizer.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Mapping, Sequence

from kvcore_amd.config.engine_config import KVCoreConfig
from kvcore_amd.sampling.params import SamplingParams

from .engine_core import EngineCore, EngineCoreOutputs
from .log import get_logger

logger = get_logger(__name__)


@dataclass(frozen=True)
class GenerationRequest:
    request_id: str
    sampling_params: SamplingParams
    messages: tuple[Mapping[str, Any], ...] | None = None
    prompt_token_ids: tuple[int, ...] | None = None


@dataclass(frozen=True)
class GenerationOutput:
    request_id: str
    output_text: str
    output_token_ids: tuple[int, ...]
    finish_reason: str | None


class LLMEngine:
    def __init__(self, kvcore_config: KVCoreConfig, *, model=None) -> None:
        self.engine_core = EngineCore(kvcore_config, model=model)

    def add_request(self, request_id: str, sampling_params: SamplingParams, *,
                    messages: Sequence[Mapping[str, Any]] | None = None,
                    prompt_token_ids: Sequence[int] | None = None) -> None:
        self.engine_core.add_request(request_id, sampling_params, messages=messages,
                                     prompt_token_ids=prompt_token_ids)

    def step(self) -> EngineCoreOutputs:
        return self.engine_core.step()

    def generate(self, requests: Sequence[GenerationRequest | Mapping[str, Any]]) -> list[GenerationOutput]:
        normalized = [self._normalize_request(r) for r in requests]
        for r in normalized:
            self.add_request(r.request_id, r.sampling_params, messages=r.messages,
                             prompt_token_ids=r.prompt_token_ids)
        while self.engine_core.has_unfinished_requests():
            out = self.step()
            state = self.engine_core.scheduler.last_no_progress_state
            if not out.request_outputs and state is not None:
                raise RuntimeError(
                    "Engine made no scheduling progress while requests are still unfinished. "
                    "This usually means the KV block budget is too small. " + state.format_message())
        outputs: list[GenerationOutput] = []
        tok = self.engine_core.tokenizer_manager
        for r in normalized:
            fin = self.engine_core.take_finished_output(r.request_id)
            if fin is None:
                continue
            outputs.append(GenerationOutput(
                request_id=r.request_id,
                output_text=tok.decode(fin.output_token_ids) if tok is not None else "",
                output_token_ids=fin.output_token_ids,
                finish_reason=None if fin.finish_reason is None else fin.finish_reason.value,
            ))
        return outputs

    @staticmethod
    def _normalize_request(request: GenerationRequest | Mapping[str, Any]) -> GenerationRequest:
        if isinstance(request, GenerationRequest):
            return request
        messages = request.get("messages")
        ids = request.get("prompt_token_ids")
        return GenerationRequest(
            request_id=request["request_id"],
            sampling_params=request["sampling_params"],
            messages=None if messages is None else tuple(messages),
            prompt_token_ids=None if ids is None else tuple(ids),
        )
