"""The step function: one batch of (request, its next tokens) through the model, from
the cache, to logits at the wanted places.

Reference: kvcore/model/model_runner.py:208-306 (``execute_model``: update states,
flatten, build metadata, forward, logits at selected rows) with kvcore/model/
input_batch.py and kvcore/kv/block_table.py.  Differences that matter:

* a request keeps its slot (its block-table row) for life, so nothing is condensed or
  moved between steps (input_batch.py:202-223 moves rows);
* one block table per cache group serves all planes of the group, and the slot of a
  token is computed inside the kernels from table and position (block_table.py:196-228
  builds a slot mapping per layer in Python);
* one packed int32 upload per step carries every index array and the block-table
  changes (model_runner.py:475-509 uploads seven tensors and 3 per layer);
* the caller says where logits are wanted; the reference takes them only at the last
  token of a request whose known tokens are all computed (model_runner.py:461-464).
"""

from __future__ import annotations

import gc
import json
import weakref
from dataclasses import dataclass, field
from pathlib import Path
from typing import Sequence

import numpy as np
import torch

from kvcore_amd.config.model_config import read_config_json
from kvcore_amd.models.decoder import DecoderModel
from kvcore_amd.ops import library as ops
from kvcore_amd.parts.base import RunLimits
from kvcore_amd.registry import resolve_architecture

from .context import CacheGroupView, StepBuffers, StepContext


@dataclass
class StepEntry:
    """One request's share of a step: ``tokens`` go to positions ``start ..``;
    ``pages[g]`` is the request's page list in cache group ``g`` (covering at least
    ``start + len(tokens)`` tokens); ``want`` lists indices into ``tokens`` whose logits
    are asked for."""

    request_id: str
    slot: int
    start: int
    tokens: Sequence[int]
    pages: Sequence[Sequence[int]]
    want: Sequence[int] = ()
    released: Sequence[int] | None = None  # per group: leading page entries that are null


@dataclass
class StepOutput:
    """``logits`` is float32 ``[S, V]`` on the device (None when nothing was wanted);
    row ``i`` belongs to ``owners[i] = (index of the entry in the step, position)``."""

    request_ids: list[str]
    logits: torch.Tensor | None
    owners: list[tuple[int, int]] = field(default_factory=list)
    num_tokens: int = 0


def build_model(model_dir: str | Path, dtype: torch.dtype, device: str | torch.device,
                *, load_format: str = "safetensors", seed: int = 0, strict: bool = True,
                config_override: dict | None = None, pack_weights: bool | None = None) -> DecoderModel:
    """config.json -> registry -> spec -> model with weights.  ``load_format="random"``
    fills the parameters from ``seed`` instead of reading weight files.  ``pack_weights``:
    see ``DecoderModel.pack_product_weights`` (None: where there is room)."""
    from kvcore_amd.weights.loader import init_random_weights, load_weights

    config = config_override if config_override is not None else read_config_json(model_dir)
    arch = resolve_architecture(config)
    typed = arch.parse_config(config)
    spec = arch.build_spec(typed)
    model = DecoderModel(spec, dtype, device)
    model.typed_config = typed
    if load_format == "random":
        init_random_weights(model, seed)
    else:
        load_weights(model, model_dir, strict=strict)
    model.packed_bytes = model.pack_product_weights(pack_weights)
    return model


class ModelRunner:
    """Owns the device side of the cache (planes, block tables, state arrays), the step
    buffers and the model; runs steps."""

    def __init__(self, model: DecoderModel, *, page_size: int | Sequence[int],
                 num_pages: int | Sequence[int], max_num_seqs: int, max_num_tokens: int,
                 max_model_len: int, use_hip_graphs: bool = True, poison_pages: bool = False) -> None:
        """``page_size`` and ``num_pages``: one value for every cache group, or one per group
        (``num_pages`` counts the null page).  ``poison_pages``: a debugging aid that fills
        every page with NaN when it is first listed for a request (see ``poison``)."""
        ops.load()  # fail here, loudly, if the kernels are not there
        if model.device.type != "cuda":
            raise RuntimeError("kvcore_amd runs on a GPU only; there is no CPU path")
        self.model = model
        self.device = model.device
        self.dtype = model.dtype
        self.max_num_seqs = max_num_seqs
        self.max_num_tokens = max_num_tokens
        self.max_model_len = max_model_len
        n_groups = len(model.cache_groups)
        self.page_sizes = [page_size] * n_groups if isinstance(page_size, int) else list(page_size)
        self.num_pages = [num_pages] * n_groups if isinstance(num_pages, int) else list(num_pages)
        if len(self.num_pages) != n_groups or len(self.page_sizes) != n_groups:
            raise ValueError("page_size and num_pages must give one value per cache group")
        self.poison_pages = poison_pages

        for gs, size in zip(model.cache_groups, self.page_sizes):
            if gs.need.page_size is not None and gs.need.page_size != size:
                raise ValueError(f"a cache group wants pages of {gs.need.page_size} tokens, got {size}")
        self.groups: list[CacheGroupView] = []
        self._allocate_cache()
        # every part learns the sizes it will run at and may refuse them now, with a message,
        # rather than in the middle of a generation
        for call in model.calls:
            limits = RunLimits(max_num_seqs, max_num_tokens, max_model_len)
            if call.group_index is not None:
                size = self.page_sizes[call.group_index]
                limits = RunLimits(max_num_seqs, max_num_tokens, max_model_len, size, -(-max_model_len // size))
            block = model.blocks[call.layer_index]
            for part in (block, *block.children().values()):
                part.check_limits(limits)
        self.states = [
            torch.zeros((max_num_seqs, *sa.need.shape), dtype=sa.need.dtype, device=self.device)
            for sa in model.state_arrays
        ]
        # a weak reference: the buffers must not keep the runner (its graphs and pinned
        # memory) alive in a cycle that only the garbage collector would free, at a time
        # of its choosing
        self_ref = weakref.ref(self)

        def drop_graphs() -> None:
            runner = self_ref()
            if runner is not None:
                runner._drop_graphs()

        self.buffers = StepBuffers(self.device, token_capacity=max_num_tokens, on_grow=drop_graphs,
                                   seq_capacity=max_num_seqs)

        # host mirror of what each slot's table rows hold: (request id, entries synced,
        # leading entries nulled) per group
        self._slot_owner: list[str | None] = [None] * max_num_seqs
        self._slot_synced = [[0] * n_groups for _ in range(max_num_seqs)]
        self._slot_released = [[0] * n_groups for _ in range(max_num_seqs)]

        # packed per-step metadata: fixed layout, one upload
        T, R = max_num_tokens, max_num_seqs
        self._upd_cap = 2 * (T + R)
        sections = [("token_ids", T), ("positions", T), ("token_req", T), ("token_rows", T),
                    ("logit_rows", T), ("q_start", R + 1), ("seq_lens", R), ("slots", R)]
        self._off: dict[str, tuple[int, int]] = {}
        cursor = 0
        for name, n in sections:
            self._off[name] = (cursor, n)
            cursor += n
        self._upd_off = cursor
        total = cursor + 3 * self._upd_cap * max(n_groups, 1)
        self._meta_host = torch.empty(total, dtype=torch.int32, pin_memory=True)
        self._meta_np = self._meta_host.numpy()
        self._meta_dev = torch.zeros(total, dtype=torch.int32, device=self.device)
        self._dev = {name: self._meta_dev[o:o + n] for name, (o, n) in self._off.items()}
        self._np = {name: self._meta_np[o:o + n] for name, (o, n) in self._off.items()}
        self._copy_done = torch.cuda.Event()
        self._copy_pending = False
        self._arange = np.arange(max(T, R) + 1, dtype=np.int32)

        # steps of single tokens are captured once per batch-size bucket and replayed
        self.use_hip_graphs = use_hip_graphs and model.graph_safe()
        self._graph_buckets = _decode_buckets(min(max_num_seqs, max_num_tokens))
        self._graphs: dict[tuple[int, int], tuple[torch.cuda.CUDAGraph, torch.Tensor]] = {}
        self._graph_warm: set[tuple[int, int]] = set()
        # one memory pool for what library calls allocate while a graph is captured (the
        # vendor matrix product's workspace): graphs never run at the same time, so they share
        self._graph_pool = None
        self.graph_replays = 0

    def _drop_graphs(self) -> None:
        """A step buffer is about to move: captured graphs hold its old address."""
        if getattr(self, "_graphs", None):
            torch.cuda.synchronize(self.device)
            self._graphs.clear()
            self._graph_warm.clear()
            self._graph_pool = None  # the pool goes with its last graph

    # -------------------------------------------------------------------- the cache
    def _allocate_cache(self) -> None:
        """Storage and block table of every cache group, as the groups' needs describe them:
        a tensor ``[entries, pages, page_size * elements a token]`` per plane of the need."""
        self.groups = []
        for gs, size, pages in zip(self.model.cache_groups, self.page_sizes, self.num_pages):
            dtype = gs.need.dtype or self.dtype
            storage = [torch.empty((gs.num_planes, pages, size * elems), dtype=dtype, device=self.device)
                       for elems in gs.need.token_elems()]
            table = torch.zeros((self.max_num_seqs, -(-self.max_model_len // size)), dtype=torch.int32,
                                device=self.device)
            self.groups.append(CacheGroupView(storage, table, size, gs.need.window))

    def resize_cache(self, num_pages: int | Sequence[int]) -> None:
        """Give the cache back and allocate it anew with ``num_pages`` pages (a value per
        group, the null page counted).  What the cache held is gone: for an engine that has
        run its profile steps on a small cache and now knows how many pages fit.  Graphs are
        dropped (they hold the old addresses), every slot is forgotten."""
        n_groups = len(self.model.cache_groups)
        self.num_pages = [num_pages] * n_groups if isinstance(num_pages, int) else list(num_pages)
        if len(self.num_pages) != n_groups:
            raise ValueError("num_pages must give one value per cache group")
        torch.cuda.synchronize(self.device)
        self._drop_graphs()
        self.groups = []  # the old storage goes before the new one comes
        torch.cuda.empty_cache()
        self._allocate_cache()
        self._slot_owner = [None] * self.max_num_seqs
        self._slot_synced = [[0] * n_groups for _ in range(self.max_num_seqs)]
        self._slot_released = [[0] * n_groups for _ in range(self.max_num_seqs)]

    # -------------------------------------------------------------------- bookkeeping
    def forget(self, slot: int) -> None:
        """A request left its slot.  The next owner's pages are synced from scratch."""
        self._slot_owner[slot] = None

    def poison(self, pages: Sequence[Sequence[int]]) -> None:
        """Fill the listed pages (one list per cache group) with NaN on the stream, behind the
        steps launched so far: for pages that were given back, so that a table row that still
        names them shows in the logits.  A debugging aid (the reference zeroes new blocks,
        kvcore/model/model_runner.py:646-657; here nothing needs it for correctness, since
        every kernel reads only the slots its request has written)."""
        for grp, ids in zip(self.groups, pages):
            ids = [p for p in ids if p > 0]
            if ids:
                dev = torch.tensor(ids, dtype=torch.int32, device=self.device)
                for plane in grp.storage:
                    ops.fill_pages(plane, dev, len(ids), float("nan"), page_axis=1)

    def fill_cache(self, value: float) -> None:
        """Overwrite every cache plane (tests fill with NaN so that a read outside a
        request's own slots shows in the logits)."""
        for g in self.groups:
            for plane in g.storage:
                plane.fill_(value)

    def cache_bytes(self) -> int:
        return sum(p.numel() * p.element_size() for g in self.groups for p in g.storage)

    def _table_updates(self, entries: Sequence[StepEntry]) -> list[list[int]]:
        """Per group, flat triples (slot, index, page) that bring the device tables up to
        the entries' page lists."""
        n_groups = len(self.groups)
        out: list[list[int]] = [[] for _ in range(n_groups)]
        for e in entries:
            slot = e.slot
            fresh = self._slot_owner[slot] != e.request_id
            if fresh:
                self._slot_owner[slot] = e.request_id
                self._slot_synced[slot] = [0] * n_groups
                self._slot_released[slot] = [0] * n_groups
            for g in range(n_groups):
                pages = e.pages[g]
                have = self._slot_synced[slot][g]
                if len(pages) > have:
                    upd = out[g]
                    for i in range(have, len(pages)):
                        upd.extend((slot, i, pages[i]))
                    self._slot_synced[slot][g] = len(pages)
                if e.released is not None:
                    done = self._slot_released[slot][g]
                    if e.released[g] > done:
                        upd = out[g]
                        for i in range(done, e.released[g]):
                            upd.extend((slot, i, 0))
                        self._slot_released[slot][g] = e.released[g]
        return out

    # --------------------------------------------------------------------------- step
    def step(self, entries: Sequence[StepEntry], device_tokens: torch.Tensor | None = None) -> StepOutput:
        """Run exactly the tokens given, as one batch, from the cache earlier steps left.
        Keys and values of these tokens are written to their pages first and read back
        from there, so what a position computes does not depend on how its request was
        cut into steps.

        ``device_tokens`` (int32 on the device, a value per entry) stands for the token ids
        of a step of single tokens whose values the host does not know yet: entry ``i``
        runs ``device_tokens[i]`` as of the time the stream gets here, and the ids in the
        entries are ignored."""
        R = len(entries)
        if R == 0:
            return StepOutput([], None)
        if R > self.max_num_seqs:
            raise ValueError(f"{R} requests in a step exceed max_num_seqs={self.max_num_seqs}")
        vocab = self.model.spec.vocab_size
        npv = self._np
        t = 0
        owners: list[tuple[int, int]] = []
        n_rows = 0
        q_lens: list[int] = []
        seq_lens: list[int] = []
        seen_slots: set[int] = set()
        if self._copy_pending:
            self._copy_done.synchronize()
            self._copy_pending = False
        decode_only = all(len(e.tokens) == 1 for e in entries)
        if device_tokens is not None:
            if not decode_only:
                raise ValueError("tokens held by the device stand for single tokens only")
            if (device_tokens.dtype != torch.int32 or device_tokens.device != self.device
                    or device_tokens.numel() < R):
                raise ValueError(f"device_tokens must hold {R} int32 values on {self.device}")
        if decode_only:
            # single tokens only: the same checks and arrays as below, without a loop of
            # array operations per request
            toks = [0] * R if device_tokens is not None else [e.tokens[0] for e in entries]
            starts = [e.start for e in entries]
            slot_list = [e.slot for e in entries]
            if min(toks) < 0 or max(toks) >= vocab:
                raise ValueError(f"a token id is outside [0, {vocab})")
            if min(starts) < 0 or max(starts) >= self.max_model_len:
                raise ValueError(f"a position exceeds max_model_len={self.max_model_len}")
            if R > self.max_num_tokens:
                raise ValueError(f"step exceeds max_num_tokens={self.max_num_tokens}")
            if min(slot_list) < 0 or max(slot_list) >= self.max_num_seqs or len(set(slot_list)) != R:
                raise ValueError("a slot is invalid or used twice")
            for e in entries:
                for g_pages, page in zip(e.pages, self.page_sizes):
                    if len(g_pages) * page <= e.start:
                        raise ValueError(f"request {e.request_id!r}: {len(g_pages)} pages do not hold "
                                         f"{e.start + 1} tokens")
            npv["token_ids"][:R] = toks
            npv["positions"][:R] = starts
            npv["token_req"][:R] = self._arange[:R]
            npv["token_rows"][:R] = slot_list
            npv["q_start"][:R + 1] = self._arange[:R + 1]
            npv["seq_lens"][:R] = starts
            npv["seq_lens"][:R] += 1
            npv["slots"][:R] = slot_list
            for r, e in enumerate(entries):
                for w in e.want:
                    if w != 0:
                        raise ValueError(f"request {e.request_id!r}: wanted index {w} outside its 1 token")
                    npv["logit_rows"][n_rows] = r
                    owners.append((r, e.start))
                    n_rows += 1
            q_lens = [1] * R
            seq_lens = [s_ + 1 for s_ in starts]
            t = R
        for r, e in enumerate(entries if not decode_only else ()):
            n = len(e.tokens)
            if n == 0:
                raise ValueError(f"request {e.request_id!r}: a step entry needs at least one token")
            end = e.start + n
            if e.start < 0 or end > self.max_model_len:
                raise ValueError(f"request {e.request_id!r}: positions {e.start}..{end - 1} exceed "
                                 f"max_model_len={self.max_model_len}")
            if t + n > self.max_num_tokens:
                raise ValueError(f"step exceeds max_num_tokens={self.max_num_tokens}")
            if not 0 <= e.slot < self.max_num_seqs or e.slot in seen_slots:
                raise ValueError(f"request {e.request_id!r}: slot {e.slot} is invalid or used twice")
            seen_slots.add(e.slot)
            for g, grp in enumerate(self.groups):
                if len(e.pages[g]) * grp.page_size < end:
                    raise ValueError(f"request {e.request_id!r}: {len(e.pages[g])} pages do not hold "
                                     f"{end} tokens")
            toks = np.asarray(e.tokens, dtype=np.int64)
            if toks.min() < 0 or toks.max() >= vocab:
                raise ValueError(f"request {e.request_id!r}: token id outside [0, {vocab})")
            npv["token_ids"][t:t + n] = toks
            npv["positions"][t:t + n] = np.arange(e.start, end, dtype=np.int32)
            npv["token_req"][t:t + n] = r
            npv["token_rows"][t:t + n] = e.slot
            npv["q_start"][r] = t
            npv["seq_lens"][r] = end
            npv["slots"][r] = e.slot
            for w in e.want:
                if not 0 <= w < n:
                    raise ValueError(f"request {e.request_id!r}: wanted index {w} outside its {n} tokens")
                npv["logit_rows"][n_rows] = t + w
                owners.append((r, e.start + w))
                n_rows += 1
            q_lens.append(n)
            seq_lens.append(end)
            t += n
        T = t
        npv["q_start"][R] = T

        # a step of single tokens that all want their logits runs padded to a bucket size,
        # so that one captured graph serves every batch of that bucket
        bucket = 0
        if self.use_hip_graphs and T == R and n_rows == R and all(w == 1 for w in q_lens):
            bucket = next((b for b in self._graph_buckets if b >= R), 0)
        if bucket:
            npv["token_ids"][R:bucket] = 0
            npv["positions"][R:bucket] = 0
            npv["token_req"][R:bucket] = -1
            npv["token_rows"][R:bucket] = -1
            npv["logit_rows"][:bucket] = np.arange(bucket, dtype=np.int32)
            npv["q_start"][R:bucket + 1] = np.arange(R, bucket + 1, dtype=np.int32)
            npv["seq_lens"][R:bucket] = 0
            npv["slots"][R:bucket] = 0

        updates = self._table_updates(entries)
        upd_counts = []
        cursor = self._upd_off
        for g, upd in enumerate(updates):
            count = len(upd) // 3
            if count > self._upd_cap:
                raise RuntimeError("block-table update overflow")  # cannot happen: bounded by pages per step
            if count:
                self._meta_np[cursor:cursor + 3 * count] = upd
            upd_counts.append((cursor, count))
            cursor += 3 * count
        self._meta_dev[:cursor].copy_(self._meta_host[:cursor], non_blocking=True)
        self._copy_done.record()
        self._copy_pending = True
        if device_tokens is not None:
            self._dev["token_ids"][:R].copy_(device_tokens[:R])
        for g, (off, count) in enumerate(upd_counts):
            if count:
                triples = self._meta_dev[off:off + 3 * count]
                ops.table_update(self.groups[g].table, triples, count)
                if self.poison_pages:  # the pages listed for the first time: third of each triple
                    for plane in self.groups[g].storage:
                        ops.fill_pages(plane, triples[2:], count, float("nan"), stride=3, page_axis=1)

        ids = [e.request_id for e in entries]
        if bucket:
            return StepOutput(ids, self._run_decode_bucket(bucket, R, max(seq_lens)), owners, T)
        ctx = self._context(T, R, q_lens, seq_lens, max(q_lens), max(seq_lens))
        hidden = self.model.forward(ctx)
        logits = None
        if n_rows:
            logits = self.model.compute_logits(ctx, hidden, self._dev["logit_rows"], n_rows)
        return StepOutput(ids, logits, owners, T)

    def _context(self, T: int, R: int, q_lens: list[int], seq_lens: list[int], max_q: int,
                 max_seq: int) -> StepContext:
        return StepContext(
            num_tokens=T, num_reqs=R,
            token_ids=self._dev["token_ids"], positions=self._dev["positions"],
            token_req=self._dev["token_req"], token_rows=self._dev["token_rows"],
            q_start=self._dev["q_start"],
            seq_lens=self._dev["seq_lens"], slots=self._dev["slots"],
            groups=self.groups, states=self.states, buffers=self.buffers,
            dtype=self.dtype, device=self.device,
            host_query_lens=q_lens, host_seq_lens=seq_lens,
            max_query_len=max_q, max_seq_len=max_seq,
        )

    def _run_decode_bucket(self, bucket: int, num_live: int, max_seq_len: int) -> torch.Tensor:
        """A padded step of ``bucket`` single tokens.  The first such step runs launch by
        launch (which also sizes every step buffer); the second is captured into a HIP
        graph; from then on the graph is replayed.  Nothing in the graph depends on the
        batch beyond what the index arrays on the device say: the context it was captured
        with claims a sequence length that bounds the batch's (the next power of two, at
        least 1024, at most the engine's limit), so that the parts may plan their launches
        by it; each such length class has a graph of its own."""
        plan_len = 1024
        while plan_len < max_seq_len:
            plan_len *= 2
        plan_len = min(plan_len, self.max_model_len)
        key = (bucket, plan_len)

        def run(keep: list | None = None) -> torch.Tensor:
            ctx = self._context(bucket, bucket, [1] * bucket, [plan_len] * bucket, 1, plan_len)
            hidden = self.model.forward(ctx)
            logits = self.model.compute_logits(ctx, hidden, self._dev["logit_rows"], bucket, every_row=True)
            if keep is not None:  # nothing made in here dies before the capture has ended
                keep.extend((ctx, hidden, logits))
            return logits

        if key in self._graphs:
            graph, logits = self._graphs[key]
            graph.replay()
            self.graph_replays += 1
            return logits[:num_live]
        if key not in self._graph_warm:
            self._graph_warm.add(key)
            return run()[:num_live]
        graph = torch.cuda.CUDAGraph()
        self.buffers.frozen = True
        # Nothing may be given back to the HIP runtime while the stream is capturing: freeing
        # pinned memory, destroying another graph or releasing its memory pool then fails, and
        # the failure ends the process.  Three guards.  (1) No garbage collection during the
        # capture (and one before it): a collection may free an earlier runner with its pinned
        # buffer and its graphs, held only by a reference cycle, at a time of its choosing.
        # (2) The step buffers are frozen: a buffer that would have to grow (which drops the
        # graphs) raises instead.  (3) What the captured step itself makes (its context, the
        # views it returns) is kept in ``keep`` until the capture has ended, so no reference
        # count reaches zero inside it.  Device memory that library calls take and give back
        # inside the capture (the vendor product's workspace) belongs to the graph's pool,
        # which the allocator does not return to the runtime while a capture runs.
        gc.collect()
        gc_was_enabled = gc.isenabled()
        gc.disable()
        keep: list = []
        try:
            if self._graph_pool is None:
                self._graph_pool = torch.cuda.graph_pool_handle()
            with torch.cuda.graph(graph, pool=self._graph_pool):
                logits = run(keep)
        finally:
            if gc_was_enabled:
                gc.enable()
            self.buffers.frozen = False
        del keep
        self._graphs[key] = (graph, logits)
        graph.replay()
        self.graph_replays += 1
        return logits[:num_live]


def _decode_buckets(limit: int) -> list[int]:
    """Batch sizes at which decode steps are captured: 1, 2, 4, 8, every size from 9 to 16
    (the products for few rows fetch every row beyond the eighth for itself, so a padded row
    costs there what a live one does, about 1% of a step each at the 8B shape; below 8 rows a
    padded row is measured to cost nothing), then steps of 8 up to 64, then steps of 32,
    always ending at the engine's limit."""
    out = [b for b in (1, 2, 4, 8, 9, 10, 11, 12, 13, 14, 15) if b < limit]
    out += list(range(16, min(limit, 64), 8))
    out += list(range(64, limit, 32))
    out.append(limit)
    return sorted(set(out))


def describe_model(model: DecoderModel) -> str:
    spec = model.spec
    return json.dumps({
        "layers": len(spec.layers), "schedule": len(spec.resolved_schedule()),
        "hidden": spec.hidden_size, "vocab": spec.vocab_size,
        "cache_groups": [(g.need.planes, g.need.window, g.num_planes)
                         for g in model.cache_groups],
        "param_bytes": model.num_param_bytes(),
    })
