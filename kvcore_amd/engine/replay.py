"""Replay of given tokens through the engine's own cache manager and step function.

A ``TraceSession`` holds a model, a ``KVManager`` and a ``ModelRunner`` and takes step
records (request id, next tokens, wanted places, requests that end).  It samples
nothing.  ``bin/trace_run`` is a thin command line over it.
"""

from __future__ import annotations

from typing import Any, Mapping

import torch

from kvcore_amd.cache.kv_manager import KVManager, plan_groups

from .runner import ModelRunner, StepEntry, StepOutput, build_model


class TraceSession:
    def __init__(self, model_dir: str, dtype: torch.dtype, *, max_tokens: int, block_size: int = 16,
                 max_num_seqs: int = 8, device: str = "cuda:0", poison_cache: bool = False,
                 shuffle_pages: int | None = None, model=None) -> None:
        self.model = model if model is not None else build_model(model_dir, dtype, device)
        page = block_size
        capacity = -(-max_tokens // 64) * 64
        self.capacity = capacity
        self.num_pages = -(-capacity // page) + 1  # + the null page
        groups = plan_groups([g.need for g in self.model.cache_groups], page, self.num_pages)
        self.manager = KVManager(groups, max_num_seqs=max_num_seqs, max_model_len=capacity,
                                 shuffle_seed=shuffle_pages, track_freed=poison_cache)
        self.runner = ModelRunner(self.model, page_size=[g.page_size for g in groups],
                                  num_pages=[g.num_pages for g in groups],
                                  max_num_seqs=max_num_seqs, max_num_tokens=capacity,
                                  max_model_len=capacity, poison_pages=poison_cache)
        if poison_cache:  # the whole cache now, every page again when it is taken or given back
            self.runner.fill_cache(float("nan"))
        self.computed: dict[str, int] = {}

    def run_step(self, record: Mapping[str, Any]) -> StepOutput | None:
        """One step record.  Returns the step's output (logits on the device, valid until
        the next step) or None when the record brought no tokens."""
        step = record.get("step")
        entries: list[StepEntry] = []
        for item in record.get("entries", []):
            rid = str(item["id"])
            tokens = [int(t) for t in item["tokens"]]
            if not tokens:
                continue
            if not self.manager.is_admitted(rid):
                self.manager.admit(rid)
                self.computed[rid] = 0
            start = self.computed[rid]
            if self.manager.allocate(rid, start, len(tokens)) is None:
                raise RuntimeError(
                    f"step {step}: request {rid!r} needs pages for {start + len(tokens)} tokens, "
                    f"free pages per group: {self.manager.num_free_pages()} of {self.num_pages - 1}; "
                    "--max-tokens is too small for this trace")
            entries.append(StepEntry(rid, self.manager.slot_of(rid), start, tokens,
                                     self.manager.page_ids(rid),
                                     [int(w) for w in item.get("want", [])],
                                     self.manager.released_counts(rid)))
        out = None
        if entries:
            if self.runner.poison_pages:
                self.runner.poison(self.manager.drain_freed())
            out = self.runner.step(entries)
            for e in entries:
                self.computed[e.request_id] += len(e.tokens)
                self.manager.release_behind_window(e.request_id, self.computed[e.request_id])
        for rid in record.get("end", []):
            rid = str(rid)
            if self.manager.is_admitted(rid):
                self.runner.forget(self.manager.slot_of(rid))
                self.manager.free(rid)
                self.computed.pop(rid, None)
        return out
