"""Per-request sampling options.

Reference: kvcore/utils/sampling_params.py:8-26 (same names, defaults and checks).
``ignore_eos`` is an addition: runs with random weights have no meaningful stop token.
"""

from __future__ import annotations

from dataclasses import dataclass


@dataclass(frozen=True)
class SamplingParams:
    max_tokens: int
    temperature: float = 1.0
    top_p: float = 1.0
    top_k: int | None = None
    seed: int | None = None
    ignore_eos: bool = False

    def __post_init__(self) -> None:
        if self.max_tokens <= 0:
            raise ValueError(f"max_tokens must be positive, got {self.max_tokens}")
        if self.temperature < 0:
            raise ValueError(f"temperature must be non-negative, got {self.temperature}")
        if not 0 < self.top_p <= 1:
            raise ValueError(f"top_p must be in (0, 1], got {self.top_p}")
        if self.top_k is not None and self.top_k <= 0:
            raise ValueError(f"top_k must be positive when set, got {self.top_k}")
