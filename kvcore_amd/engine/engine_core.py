"""Wires model, cache manager, scheduler, runner and sampler; runs engine steps.

Reference: kvcore/engine/engine_core.py:37-217 (construction order, ``add_request``,
``step`` = schedule, execute, sample, update; stop ids from tokenizer and config) and
kvcore/model/model_runner.py:131-163,691-768 (how many pages fit).
"""

from __future__ import annotations

import time
from dataclasses import dataclass
from typing import Any, Mapping, Sequence

import torch

from kvcore_amd.cache.kv_manager import KVManager, cdiv, plan_groups
from kvcore_amd.config.engine_config import KVCoreConfig, canonical_dtype
from kvcore_amd.config.model_config import read_config_json, read_generation_eos
from kvcore_amd.sampling.params import SamplingParams
from kvcore_amd.sampling.sampler import PendingTokens, Sampler, SamplingRow

from .log import get_logger
from .request import FinishReason, Request
from .runner import ModelRunner, StepEntry, build_model
from .scheduler import RequestStepOutput, Scheduler, SchedulerOutput
from .tokenizer import TokenizerManager

logger = get_logger(__name__)

TORCH_DTYPES = {"bfloat16": torch.bfloat16, "float32": torch.float32}


@dataclass(frozen=True)
class EngineCoreOutputs:
    request_outputs: tuple[RequestStepOutput, ...] = ()


@dataclass(frozen=True)
class FinishedRequestOutput:
    request_id: str
    output_token_ids: tuple[int, ...]
    finish_reason: FinishReason | None


@dataclass
class StepStats:
    """Wall-clock seconds of the last step's parts (the reference keeps the same in
    ``ModelRunnerStepStats``, model_runner.py:81-91); the forward time includes the
    wait for the GPU, because sampling ends in a synchronisation."""

    schedule: float = 0.0
    forward_and_sample: float = 0.0
    update: float = 0.0
    num_tokens: int = 0
    num_reqs: int = 0


def resolve_dtype(config: KVCoreConfig, model_json: Mapping[str, Any]) -> torch.dtype:
    """ModelConfig.dtype, else config.json's ``dtype`` if it is one of ours, else
    bfloat16 (reference: model_loader/utils.py:10-16 falls back to torch's default)."""
    name = config.model_config.dtype
    if name is None:
        raw = model_json.get("dtype", model_json.get("torch_dtype"))
        try:
            name = canonical_dtype(raw)
        except ValueError:
            name = None
    return TORCH_DTYPES[name or "bfloat16"]


class EngineCore:
    def __init__(self, config: KVCoreConfig, *, model=None) -> None:
        self.config = config
        device = torch.device(config.device_config.device)
        model_json = read_config_json(config.model_config.model) if model is None else {}
        self.dtype = resolve_dtype(config, model_json) if model is None else model.dtype
        t0 = time.perf_counter()
        if model is None:
            fmt = config.load_config.load_format
            model = build_model(config.model_config.model, self.dtype, device,
                                load_format="random" if fmt == "random" else "safetensors",
                                seed=config.load_config.seed, strict=config.load_config.strict,
                                pack_weights=config.load_config.pack_decode_weights)
        self.model = model
        logger.info("model ready in %.2f s (%d parameter bytes, %d more in packed copies)",
                    time.perf_counter() - t0, model.num_param_bytes(), getattr(model, "packed_bytes", 0))

        sched = config.scheduler_config
        cache = config.cache_config
        self.max_model_len = config.model_config.max_model_len or model.spec.max_position_embeddings
        self.page_size = cache.block_size
        # ``num_pages`` counts pages of ``block_size`` tokens (with the null page); a cache
        # group whose mixers want another page size holds the same number of tokens
        self.num_pages = self._decide_num_pages()
        self.group_configs = plan_groups([g.need for g in model.cache_groups], self.page_size, self.num_pages)
        self.kv_manager = KVManager(self.group_configs, max_num_seqs=sched.max_num_seqs,
                                    max_model_len=self.max_model_len, track_freed=cache.poison_pages)
        self.scheduler = Scheduler(sched, self.kv_manager, max_model_len=self.max_model_len)
        self.runner = ModelRunner(model, page_size=[g.page_size for g in self.group_configs],
                                  num_pages=[g.num_pages for g in self.group_configs],
                                  max_num_seqs=sched.max_num_seqs,
                                  max_num_tokens=sched.max_num_scheduled_tokens,
                                  max_model_len=self.max_model_len,
                                  use_hip_graphs=config.device_config.use_hip_graphs,
                                  poison_pages=cache.poison_pages)
        if cache.poison_pages:
            self.runner.fill_cache(float("nan"))
        self.sampler = Sampler(device, sched.max_num_seqs, engine_seed=config.load_config.seed)
        self.tokenizer_manager = None
        if model_json:
            self.tokenizer_manager = TokenizerManager.from_model_source(
                config.model_config.tokenizer or config.model_config.model)
        # stop ids: config.json's, generation_config.json's and the tokenizer's, joined
        # (reference: engine_core.py:209-217 joins the tokenizer's and the config's)
        self.stop_token_ids = set(model.spec.eos_token_ids)
        if model_json:
            self.stop_token_ids |= set(read_generation_eos(config.model_config.model))
        if self.tokenizer_manager is not None:
            self.stop_token_ids |= self.tokenizer_manager.get_stop_token_ids()
        self._seeds: dict[str, int] = {}
        self.run_ahead = sched.decode_run_ahead and model.device.type == "cuda"
        self._in_flight: _Flight | None = None
        self._finished: dict[str, FinishedRequestOutput] = {}
        self.last_step_stats = StepStats()

    # ---------------------------------------------------------------------- capacity
    def bytes_per_page(self) -> int:
        """Bytes that ``block_size`` tokens take in the cache, over all groups and planes."""
        return sum(g.num_planes * 2 * g.need.num_kv_heads * self.page_size * g.need.head_dim
                   * torch.empty((), dtype=g.need.dtype or self.dtype).element_size()
                   for g in self.model.cache_groups)

    def _decide_num_pages(self) -> int:
        """An explicit ``num_gpu_blocks`` wins.  Otherwise: free device memory times the
        utilisation, minus an estimate of the step buffers and a fixed margin, divided by
        the bytes of one page over all planes; never more than every slot at full length
        needs (reference: model_runner.py:696-768 measures the activation peak with a
        dummy forward; the buffers here have known sizes)."""
        cache = self.config.cache_config
        sched = self.config.scheduler_config
        if cache.num_gpu_blocks is not None:
            return cache.num_gpu_blocks
        per_page = max(self.bytes_per_page(), 1)
        useful = sched.max_num_seqs * cdiv(self.max_model_len, self.page_size) + 1
        if not cache.profile_kv_cache or self.model.device.type != "cuda":
            return useful
        free, total = torch.cuda.mem_get_info(self.model.device)
        esize = torch.empty((), dtype=self.dtype).element_size()
        spec = self.model.spec
        widest = max((p.shape[0] for bp in self.model.params.values() for p in [bp.spec]
                      if len(bp.spec.shape) == 2 and bp.spec.shape[0] != spec.vocab_size), default=spec.hidden_size)
        per_token = 4 * spec.hidden_size + esize * (4 * spec.hidden_size + 3 * widest)
        activations = sched.max_num_scheduled_tokens * per_token
        activations += sched.max_num_seqs * spec.vocab_size * (4 + esize)
        margin = 512 << 20
        budget = min(total * cache.gpu_memory_utilization - (total - free), free) - activations - margin
        pages = int(budget // per_page)
        if pages < 2:
            raise RuntimeError(
                f"not enough device memory for a KV cache: {free / 2**30:.1f} GiB free, "
                f"{activations / 2**30:.2f} GiB of step buffers, {per_page} bytes per page")
        return min(pages, useful)

    # ---------------------------------------------------------------------- requests
    def add_request(self, request_id: str, sampling_params: SamplingParams, *,
                    messages: Sequence[Mapping[str, Any]] | None = None,
                    prompt_token_ids: Sequence[int] | None = None) -> None:
        if prompt_token_ids is None:
            if messages is None:
                raise ValueError("a request needs messages or prompt_token_ids")
            if self.tokenizer_manager is None:
                raise ValueError("the model folder has no tokenizer; give prompt_token_ids")
            prompt_token_ids = self.tokenizer_manager.encode_messages(messages)
        vocab = self.model.spec.vocab_size
        if any(not 0 <= int(t) < vocab for t in prompt_token_ids):
            raise ValueError(f"request {request_id!r}: a prompt token id is outside [0, {vocab})")
        request = Request(request_id, [int(t) for t in prompt_token_ids], sampling_params)
        self.scheduler.add_request(request)
        self._seeds[request_id] = self.sampler.resolve_seed(sampling_params)

    def has_unfinished_requests(self) -> bool:
        return self.scheduler.has_unfinished_requests()

    def take_finished_output(self, request_id: str) -> FinishedRequestOutput | None:
        return self._finished.pop(request_id, None)

    def abort_requests(self, request_ids: Sequence[str] | None = None) -> None:
        from .request import RequestStatus

        for state in self.scheduler.finish_requests(request_ids, RequestStatus.FINISHED_ABORTED):
            self._finished[state.request_id] = FinishedRequestOutput(
                state.request_id, state.output_token_ids, state.finish_reason)
            self._seeds.pop(state.request_id, None)
        flight, self._in_flight = self._in_flight, None
        if flight is not None:
            self._keep_in_flight(flight)

    # -------------------------------------------------------------------------- step
    def step(self) -> EngineCoreOutputs:
        """One model step's results.  While requests only decode, the step after the one
        whose results are returned is already running (see ``_launch_ahead``)."""
        stats = StepStats()
        t0 = time.perf_counter()
        flight = self._in_flight
        self._in_flight = None
        if flight is None:
            out = self.scheduler.schedule()
            stats.schedule = time.perf_counter() - t0
            if out.is_empty:
                self.last_step_stats = stats
                return EngineCoreOutputs()
            flight = self._launch(out)
        out = flight.output
        t1 = time.perf_counter()
        ahead = self._launch_ahead(flight) if self.run_ahead else None
        sampled = dict(zip(flight.row_ids, flight.tokens.result()))
        t2 = time.perf_counter()
        stats.forward_and_sample = t2 - t1
        result = self.scheduler.update_from_outputs(out, sampled, stop_token_ids=self.stop_token_ids)
        for state in result.finished_requests:
            self._finished[state.request_id] = FinishedRequestOutput(
                state.request_id, state.output_token_ids, state.finish_reason)
            self._seeds.pop(state.request_id, None)
        if ahead is not None:
            self._keep_in_flight(ahead)
        stats.update = time.perf_counter() - t2
        stats.num_tokens = out.total_num_scheduled_tokens
        stats.num_reqs = len(out.scheduled)
        self.last_step_stats = stats
        logger.info("step %d: %d requests, %d tokens, schedule %.2f ms, forward+sample %.2f ms",
                    out.step_id, stats.num_reqs, stats.num_tokens, stats.schedule * 1e3,
                    stats.forward_and_sample * 1e3)
        return EngineCoreOutputs(result.step_outputs)

    def execute(self, out: SchedulerOutput) -> dict[str, int]:
        """Run one scheduled step and sample where a request's known tokens end."""
        flight = self._launch(out)
        return dict(zip(flight.row_ids, flight.tokens.result()))

    def _launch(self, out: SchedulerOutput, device_tokens: torch.Tensor | None = None) -> "_Flight":
        """Launch a scheduled step and its sampling; wait for nothing."""
        entries = []
        rows: list[SamplingRow] = []
        row_ids: list[str] = []
        for s in out.scheduled:
            if s.is_new:
                self.runner.forget(s.slot)
            n = len(s.token_ids)
            entries.append(StepEntry(s.request_id, s.slot, s.num_computed_tokens, s.token_ids,
                                     s.page_ids, (n - 1,) if s.samples else (), s.released))
            if s.samples:
                rows.append(SamplingRow(s.sampling_params, self._seeds[s.request_id], s.num_output_tokens))
                row_ids.append(s.request_id)
        if self.runner.poison_pages:
            self.runner.poison(self.kv_manager.drain_freed())
        step_out = self.runner.step(entries, device_tokens)
        tokens = self.sampler.launch(step_out.logits, rows) if rows else PendingTokens(None, 0)
        return _Flight(out, row_ids, tokens)

    def _launch_ahead(self, flight: "_Flight") -> "_Flight | None":
        """Before the tokens of the step in flight are awaited: if the scheduler can say what
        the next step is without them (requests that only decode), launch it behind the one
        in flight, each request's token being read from where that one's sampling leaves it.
        The host's work for a step then overlaps the device's work for the step before.  A
        request that turns out to have ended on a stop token has run one token too many,
        which is dropped (``_keep_in_flight``).  Its key and value land in a page that the
        host has given back by then; on the device that write comes before anything a later
        owner of the page does, and an owner reads only the slots it has written itself."""
        if flight.row_ids != [s.request_id for s in flight.output.scheduled]:
            return None  # a request was dropped from it: its rows are not the next step's rows
        planned = self.scheduler.plan_decode_ahead(flight.output)
        if planned is None:
            return None
        return self._launch(planned, flight.tokens.device)

    def _keep_in_flight(self, flight: "_Flight") -> None:
        """The step launched ahead becomes the step in flight, without the requests that
        have ended meanwhile."""
        out = self.scheduler.without_finished(flight.output)
        if out.is_empty:
            return
        if out is not flight.output:
            flight = _Flight(out, flight.row_ids, flight.tokens)
        self._in_flight = flight


@dataclass
class _Flight:
    """A launched step: what was scheduled, the requests of the sampled rows in row order
    (all of them, also those dropped from ``output`` since) and the tokens on their way."""

    output: SchedulerOutput
    row_ids: list[str]
    tokens: PendingTokens
