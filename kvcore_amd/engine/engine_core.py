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


@dataclass(frozen=True)
class MemoryProfile:
    """What the profile steps measured, in bytes, and the page count that follows."""

    total: int
    free: int
    others: int  # held on the device by anything but torch's allocator
    live: int  # tensors that stay: weights, step buffers, workspaces, the graphs' pool
    transient: int  # what a step takes and gives back
    margin: int
    budget: int
    bytes_per_page: int
    pages: int
    useful_pages: int
    formula_pages: int


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


def join_stop_token_ids(config_eos, model_dir, tokenizer_manager) -> set[int]:
    """The ids that end a request: config.json's ``eos_token_id``, the tokenizer's, and those
    of the folder's generation_config.json.  The reference joins the first two
    (engine_core.py:209-217); the third is this engine's addition, on purpose: instruct
    checkpoints of Llama 3 name their end-of-turn id only there, and without it a chat request
    runs to its length cap.  A folder whose generation_config.json lists further ids therefore
    stops on them here and would not in the reference."""
    stop = set(config_eos)
    if model_dir is not None:
        stop |= set(read_generation_eos(model_dir))
    if tokenizer_manager is not None:
        stop |= tokenizer_manager.get_stop_token_ids()
    return stop


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
        self.sampler = Sampler(device, sched.max_num_seqs, engine_seed=config.load_config.seed)
        # ``num_pages`` counts pages of ``block_size`` tokens (with the null page); a cache
        # group whose mixers want another page size holds the same number of tokens.  With no
        # count given, the runner is built on a cache just large enough for the profile steps,
        # which tell how much room is left, and the cache is then allocated anew
        self.memory_profile: MemoryProfile | None = None
        profiled = (cache.num_gpu_blocks is None and cache.profile_kv_cache and model.device.type == "cuda"
                    and bool(model.cache_groups))
        first_pages = self._profile_pages() if profiled else self._pages_without_profile()
        first_groups = plan_groups([g.need for g in model.cache_groups], self.page_size, first_pages)
        self.runner = ModelRunner(model, page_size=[g.page_size for g in first_groups],
                                  num_pages=[g.num_pages for g in first_groups],
                                  max_num_seqs=sched.max_num_seqs,
                                  max_num_tokens=sched.max_num_scheduled_tokens,
                                  max_model_len=self.max_model_len,
                                  use_hip_graphs=config.device_config.use_hip_graphs,
                                  poison_pages=cache.poison_pages)
        self.num_pages = first_pages
        self.group_configs = first_groups
        if profiled:
            self.num_pages = self._measure_num_pages()
            self.group_configs = plan_groups([g.need for g in model.cache_groups], self.page_size, self.num_pages)
            self.runner.resize_cache([g.num_pages for g in self.group_configs])
        self.kv_manager = KVManager(self.group_configs, max_num_seqs=sched.max_num_seqs,
                                    max_model_len=self.max_model_len, track_freed=cache.poison_pages)
        self.scheduler = Scheduler(sched, self.kv_manager, max_model_len=self.max_model_len)
        if cache.poison_pages:
            self.runner.fill_cache(float("nan"))
        self.tokenizer_manager = None
        if model_json:
            self.tokenizer_manager = TokenizerManager.from_model_source(
                config.model_config.tokenizer or config.model_config.model)
        self.stop_token_ids = join_stop_token_ids(
            model.spec.eos_token_ids, config.model_config.model if model_json else None,
            self.tokenizer_manager)
        self._seeds: dict[str, int] = {}
        self.run_ahead = sched.decode_run_ahead and model.device.type == "cuda"
        self._in_flight: _Flight | None = None
        self._finished: dict[str, FinishedRequestOutput] = {}
        self.last_step_stats = StepStats()

    # ---------------------------------------------------------------------- capacity
    def bytes_per_page(self) -> int:
        """Bytes that ``block_size`` tokens take in the cache, over all groups, entries and
        planes (what a group keeps per token is its need's ``planes``)."""
        return sum(g.num_planes * sum(g.need.token_elems()) * self.page_size
                   * torch.empty((), dtype=g.need.dtype or self.dtype).element_size()
                   for g in self.model.cache_groups)

    def useful_pages(self) -> int:
        """More pages than this no traffic can hold: every slot at the longest length."""
        return self.config.scheduler_config.max_num_seqs * cdiv(self.max_model_len, self.page_size) + 1

    def _pages_without_profile(self) -> int:
        cache = self.config.cache_config
        return cache.num_gpu_blocks if cache.num_gpu_blocks is not None else self.useful_pages()

    def _profile_pages(self) -> int:
        """Pages of the cache that the profile steps run on: room for one step's tokens."""
        sched = self.config.scheduler_config
        return min(self.useful_pages(), cdiv(sched.max_num_scheduled_tokens, self.page_size) + 2)

    def _run_profile_steps(self) -> None:
        """The largest step of each kind on the engine's own runner and sampler, so that every
        step buffer, workspace and graph pool is there at its largest: a step of
        ``max_num_scheduled_tokens`` prompt tokens (in as few requests as ``max_model_len``
        allows), sampled both ways, then a step of single tokens for every slot, three times
        (launch by launch, captured, replayed).  Pages are dealt round and round from the small
        cache: what the steps compute is thrown away."""
        sched = self.config.scheduler_config
        runner = self.runner
        counters = [0] * len(runner.groups)

        def pages_for(tokens: int) -> list[list[int]]:
            out = []
            for g, grp in enumerate(runner.groups):
                ids = []
                for _ in range(cdiv(tokens, grp.page_size)):
                    ids.append(1 + counters[g] % (grp.num_pages - 1))
                    counters[g] += 1
                out.append(ids)
            return out

        def sample_both_ways(logits: torch.Tensor) -> None:
            n = logits.shape[0]
            greedy = SamplingParams(max_tokens=1, temperature=0.0)
            drawn = SamplingParams(max_tokens=1, temperature=1.0, top_k=50, top_p=0.9)
            self.sampler.launch(logits, [SamplingRow(greedy, 0, 0)] * n).result()
            self.sampler.launch(logits, [SamplingRow(drawn, i, 0) for i in range(n)]).result()

        left = sched.max_num_scheduled_tokens
        entries = []
        while left > 0 and len(entries) < sched.max_num_seqs:
            n = min(left, self.max_model_len)
            slot = len(entries)
            entries.append(StepEntry(f"profile-p{slot}", slot, 0, [0] * n, pages_for(n), (n - 1,)))
            left -= n
        sample_both_ways(runner.step(entries).logits)
        singles = min(sched.max_num_seqs, sched.max_num_scheduled_tokens)
        entries = [StepEntry(f"profile-d{slot}", slot, 0, [0], pages_for(1), (0,)) for slot in range(singles)]
        for _ in range(3):
            sample_both_ways(runner.step(entries).logits)

    def _measure_num_pages(self) -> int:
        """How many pages fit, by measurement (reference: model_runner.py:696-768 runs a dummy
        forward at ``max_num_scheduled_tokens``, reads torch's peak and gives the cache what
        ``gpu_memory_utilization`` of the device leaves beside it).  Here the profile steps run
        on the engine's own runner, so what they allocate stays and is counted as it is:
        ``live`` (weights, step buffers, workspaces, the graphs' pool), plus ``transient``, what
        a step takes and gives back, plus what others hold on the device.  Never more than
        every slot at full length needs.  The estimate by formula that stood here before is
        logged beside the measurement."""
        cache = self.config.cache_config
        device = self.model.device
        per_page = max(self.bytes_per_page(), 1)
        torch.cuda.synchronize(device)
        torch.cuda.reset_peak_memory_stats(device)
        self._run_profile_steps()
        torch.cuda.synchronize(device)
        peak = torch.cuda.max_memory_allocated(device)
        now = torch.cuda.memory_allocated(device)
        live = now - self.runner.cache_bytes()
        transient = max(peak - now, 0)
        free, total = torch.cuda.mem_get_info(device)
        others = max((total - free) - torch.cuda.memory_reserved(device), 0)
        margin = 512 << 20  # for graphs of further batch sizes and what the allocator cannot pack
        budget = int(total * cache.gpu_memory_utilization) - others - live - transient - margin
        pages = int(budget // per_page)
        useful = self.useful_pages()
        formula = self._estimate_num_pages_by_formula(free + self.runner.cache_bytes(), total)
        self.memory_profile = MemoryProfile(total, free, others, live, transient, margin, budget, per_page,
                                            min(pages, useful), useful, formula)
        logger.info("KV cache by measurement: total %.2f GiB, others %.2f, live %.2f, transient %.2f, "
                    "margin %.2f, budget %.2f GiB, %d bytes a page -> %d pages (useful %d; the formula "
                    "says %d, off by %+.1f%%)", total / 2**30, others / 2**30, live / 2**30,
                    transient / 2**30, margin / 2**30, budget / 2**30, per_page, pages, useful, formula,
                    100.0 * (formula - pages) / max(pages, 1))
        if pages < 2:
            raise RuntimeError(
                f"not enough device memory for a KV cache: {total / 2**30:.1f} GiB in all, "
                f"{(others + live + transient) / 2**30:.2f} GiB taken by weights, step buffers and "
                f"others, {per_page} bytes per page")
        return min(pages, useful)

    def _estimate_num_pages_by_formula(self, free: int, total: int) -> int:
        """The cross-check: step buffers guessed from the model's widths."""
        cache = self.config.cache_config
        sched = self.config.scheduler_config
        esize = torch.empty((), dtype=self.dtype).element_size()
        spec = self.model.spec
        widest = max((p.shape[0] for bp in self.model.params.values() for p in [bp.spec]
                      if len(bp.spec.shape) == 2 and bp.spec.shape[0] != spec.vocab_size), default=spec.hidden_size)
        per_token = 4 * spec.hidden_size + esize * (4 * spec.hidden_size + 3 * widest)
        activations = sched.max_num_scheduled_tokens * per_token
        activations += sched.max_num_seqs * spec.vocab_size * (4 + esize)
        budget = min(total * cache.gpu_memory_utilization - (total - free), free) - activations - (512 << 20)
        return int(budget // max(self.bytes_per_page(), 1))

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
