"""Turns float32 logits into token ids on the GPU.

Reference: kvcore/sample/sampler.py:86-167: float logits; rows whose temperature is
below 1e-5 take the argmax; the others are divided by their temperature, filtered by
top-k and top-p, and drawn as ``argmax(softmax / q)`` with ``q ~ Exp(1)``.  The
reference seeds a fresh generator inside every call (:53-57,185-188), so a seeded
request would draw the same noise for every token; here the noise of a request's
``index``-th output token is a function of (seed, index) alone, so a seeded run is
reproducible, independent of what else is in the batch, and fresh at every token.
"""

from __future__ import annotations

import os
from dataclasses import dataclass
from typing import Sequence

import numpy as np
import torch

from kvcore_amd.ops import library as ops

from .params import SamplingParams

GREEDY_EPS = 1e-5  # sampler.py:11


@dataclass(frozen=True)
class SamplingRow:
    """One logits row's options: ``seed`` is the request's 64-bit seed (already
    resolved), ``index`` the number of tokens the request has produced so far."""

    params: SamplingParams
    seed: int
    index: int


class _Lane:
    """Buffers of one sampling call: options on host and device, tokens on device and host."""

    def __init__(self, n: int, device: torch.device) -> None:
        self.host = torch.empty(6 * n, dtype=torch.int32, pin_memory=True)
        self.host_np = self.host.numpy()
        self.dev = torch.empty(6 * n, dtype=torch.int32, device=device)
        self.out_dev = torch.empty(n, dtype=torch.int32, device=device)
        self.out_host = torch.empty(n, dtype=torch.int32, pin_memory=True)
        self.done = torch.cuda.Event()


class PendingTokens:
    """Tokens of a sampling call that has been launched: ``device`` holds them as soon as
    the stream gets there, ``result()`` waits for their copy on the host."""

    def __init__(self, lane: _Lane | None, count: int) -> None:
        self._lane = lane
        self.count = count
        self.device = None if lane is None else lane.out_dev[:count]

    def result(self) -> list[int]:
        if self._lane is None:
            return []
        self._lane.done.synchronize()
        return self._lane.out_host[:self.count].tolist()


class Sampler:
    def __init__(self, device: torch.device | str, max_rows: int, engine_seed: int | None = None) -> None:
        self.device = torch.device(device)
        self.max_rows = max_rows
        self.engine_seed = int.from_bytes(os.urandom(8), "little") if engine_seed is None else engine_seed
        self._requests_seen = 0
        # two sets of buffers, used in turn: a step may be launched while the tokens of the
        # step before are still on their way to the host
        self._lanes = [_Lane(max_rows, self.device) for _ in range(2)]
        self._turn = 0
        self._part_val: torch.Tensor | None = None  # workspace of the two-stage argmax
        self._part_idx: torch.Tensor | None = None
        self._workspace: torch.Tensor | None = None  # lets several blocks sample one row

    def resolve_seed(self, params: SamplingParams) -> int:
        """The request's own seed, or one derived from the engine's seed and the order of
        arrival (the reference draws unseeded rows from torch's global generator)."""
        self._requests_seen += 1
        if params.seed is not None:
            return params.seed & 0xFFFFFFFFFFFFFFFF
        x = (self.engine_seed + 0x9E3779B97F4A7C15 * self._requests_seen) & 0xFFFFFFFFFFFFFFFF
        x ^= x >> 31
        return (x * 0xBF58476D1CE4E5B9) & 0xFFFFFFFFFFFFFFFF

    def sample(self, logits: torch.Tensor, rows: Sequence[SamplingRow]) -> list[int]:
        return self.launch(logits, rows).result()

    def launch(self, logits: torch.Tensor, rows: Sequence[SamplingRow]) -> PendingTokens:
        """Launch the sampling of ``rows`` and the copy of the tokens to the host; wait for
        neither.  At most two calls may be pending: the third reuses the first's buffers."""
        S = len(rows)
        if logits.shape[0] != S:
            raise ValueError(f"{S} sampling rows for {logits.shape[0]} logits rows")
        if S == 0:
            return PendingTokens(None, 0)
        if S > self.max_rows:
            raise ValueError(f"{S} rows exceed the sampler's capacity {self.max_rows}")
        lane = self._lanes[self._turn]
        self._turn ^= 1
        out = lane.out_dev[:S]
        if all(r.params.temperature < GREEDY_EPS for r in rows):
            need = S * (-(-logits.shape[1] // 8192))
            if self._part_val is None or self._part_val.numel() < need:
                self._part_val = torch.empty(max(need, self.max_rows), dtype=torch.float32, device=self.device)
                self._part_idx = torch.empty(max(need, self.max_rows), dtype=torch.int32, device=self.device)
            ops.argmax(out, logits, self._part_val, self._part_idx)
        else:
            n = self.max_rows
            buf = lane.host_np
            fview = buf.view(np.float32)
            uview = buf.view(np.uint32)
            V = logits.shape[1]
            filters = 0
            for i, r in enumerate(rows):
                p = r.params
                fview[i] = p.temperature
                buf[n + i] = 0 if p.top_k is None else min(p.top_k, V)
                fview[2 * n + i] = p.top_p
                if p.temperature >= GREEDY_EPS:
                    filters |= (1 if p.top_k is not None and 0 < p.top_k < V else 0) | (2 if p.top_p < 1.0 else 0)
                uview[3 * n + i] = r.seed & 0xFFFFFFFF
                uview[4 * n + i] = (r.seed >> 32) & 0xFFFFFFFF
                uview[5 * n + i] = r.index & 0xFFFFFFFF
            lane.dev.copy_(lane.host, non_blocking=True)
            d = lane.dev
            words = ops.sample_workspace_words(S, V)
            if words and (self._workspace is None or self._workspace.numel() < words):
                self._workspace = torch.empty(max(words, ops.sample_workspace_words(min(n, 64), V)),
                                              dtype=torch.int64, device=self.device)
            ops.sample(out, logits, temperature=d[:n].view(torch.float32), top_k=d[n:2 * n],
                       top_p=d[2 * n:3 * n].view(torch.float32), seed_lo=d[3 * n:4 * n],
                       seed_hi=d[4 * n:5 * n], index=d[5 * n:6 * n],
                       workspace=self._workspace if words else None, filters=filters)
        lane.out_host[:S].copy_(out, non_blocking=True)
        lane.done.record()
        return PendingTokens(lane, S)
