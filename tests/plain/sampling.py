"""Plain sampling: the reference's formulas on whole rows, in float64, on the CPU.

Shares no code with the product.  The noise is the one thing both sides must agree
on bit for bit, so its recipe is written out here a second time from its
description: 32-bit integer mixing of (seed, output index, vocabulary index), the
top 23 bits plus a half taken as a uniform number in (0, 1), minus its logarithm as an
exponential variate.
"""

from __future__ import annotations

import math

import torch

SAMPLING_EPS = 1e-5  # reference: kvcore/sample/sampler.py:11

_M32 = 0xFFFFFFFF


def _fmix(x: int) -> int:
    x &= _M32
    x ^= x >> 16
    x = (x * 0x85EBCA6B) & _M32
    x ^= x >> 13
    x = (x * 0xC2B2AE35) & _M32
    x ^= x >> 16
    return x


def noise_key(seed: int, index: int) -> int:
    lo = seed & _M32
    hi = (seed >> 32) & _M32
    key = _fmix(lo ^ _fmix((hi + 0x9E3779B9) & _M32))
    return _fmix(key ^ _fmix((index + 0x7F4A7C15) & _M32))


def uniform_noise(seed: int, index: int, vocab: int) -> torch.Tensor:
    """``u[v]`` in (0, 1) for one (seed, output index)."""
    key = noise_key(seed, index)
    out = torch.empty(vocab, dtype=torch.float64)
    for v in range(vocab):
        x = _fmix((key + v * 0x9E3779B1) & _M32)
        x = _fmix(x ^ key)
        out[v] = ((x >> 9) + 0.5) / 8388608.0
    return out


def exponential_noise(seed: int, index: int, vocab: int) -> torch.Tensor:
    return -torch.log(uniform_noise(seed, index, vocab))


def greedy(logits: torch.Tensor) -> int:
    """Reference: sampler.py:118-119."""
    return int(torch.argmax(logits))


def apply_top_k_top_p(logits: torch.Tensor, top_k: int | None, top_p: float | None) -> torch.Tensor:
    """One row.  Reference: sampler.py:132-155: ascending sort; values below the k-th
    largest are masked; then, over the softmax of what is left, entries whose
    cumulative sum from the small end is ``<= 1 - p`` are masked, the largest never."""
    if top_k is None and top_p is None:
        return logits
    V = logits.numel()
    sorted_vals, sorted_idx = torch.sort(logits, descending=False)
    if top_k is not None:
        k = min(top_k, V)
        threshold = sorted_vals[V - k]
        sorted_vals = sorted_vals.masked_fill(sorted_vals < threshold, -math.inf)
    if top_p is not None:
        probs = torch.softmax(sorted_vals, dim=-1)
        cum = torch.cumsum(probs, dim=-1)
        mask = cum <= 1 - top_p
        mask[-1] = False
        sorted_vals = sorted_vals.masked_fill(mask, -math.inf)
    out = torch.empty_like(logits)
    out[sorted_idx] = sorted_vals
    return out


def sample(
    logits: torch.Tensor,
    *,
    temperature: float,
    top_k: int | None = None,
    top_p: float = 1.0,
    seed: int = 0,
    index: int = 0,
) -> int:
    """One row.  Reference: sampler.py:86-115 (float logits; greedy below 1e-5;
    divide by the temperature; top-k/top-p; softmax; ``argmax(probs / q)`` with
    ``q ~ Exp(1)``, :158-167).  The reference seeds a fresh generator at every call;
    here the noise of output token ``index`` is a function of (seed, index)."""
    logits = logits.to(torch.float64)
    if temperature < SAMPLING_EPS:
        return greedy(logits)
    logits = logits / temperature
    logits = apply_top_k_top_p(logits, top_k, None if top_p >= 1.0 else top_p)
    probs = torch.softmax(logits, dim=-1)
    q = exponential_noise(seed, index, logits.numel())
    return int(torch.argmax(probs / q))
