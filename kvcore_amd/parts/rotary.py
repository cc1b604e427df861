"""Rotary position encoding: a frequency table, optionally rescaled, and per-step
cos/sin tables computed once in float32 and shared by every layer.

Reference: kvcore/model/layer/rotary_embedding.py:52-98: ``inv_freq[j] = base **
(-2j/d)``, angles ``position * inv_freq`` in float32, element ``j`` paired with
``j + d/2``.  The reference rounds cos and sin to the model dtype before the multiply
(:95-96); here the rotation itself is float32 and only its result is rounded.  The
``llama3`` frequency rescaling has no counterpart in the reference.
"""

from __future__ import annotations

import math

import torch

from kvcore_amd.ops import library as ops

from .base import PositionEncoding, RotaryTables, register_position_encoding


def rotary_inv_freq(rot_dim: int, theta: float, scaling: dict | None = None) -> torch.Tensor:
    """float32 ``[rot_dim / 2]``.  ``scaling`` None or ``{"rope_type": "default"}`` is the
    plain table; ``{"rope_type": "llama3", factor, low_freq_factor, high_freq_factor,
    original_max_position_embeddings}`` divides long wavelengths by ``factor``, keeps
    short ones and blends linearly (in original_length / wavelength) between the two."""
    exponents = torch.arange(0, rot_dim, 2, dtype=torch.float64) / rot_dim
    inv_freq = 1.0 / (torch.tensor(float(theta), dtype=torch.float64) ** exponents)
    rope_type = "default" if not scaling else scaling.get("rope_type", "default")
    if rope_type == "llama3":
        factor = float(scaling["factor"])
        low = float(scaling["low_freq_factor"])
        high = float(scaling["high_freq_factor"])
        orig = float(scaling["original_max_position_embeddings"])
        wavelen = 2.0 * math.pi / inv_freq
        smooth = ((orig / wavelen - low) / (high - low)).clamp(0.0, 1.0)
        blended = (1.0 - smooth) * inv_freq / factor + smooth * inv_freq
        inv_freq = torch.where(wavelen < orig / high, inv_freq,
                               torch.where(wavelen > orig / low, inv_freq / factor, blended))
    elif rope_type != "default":
        raise ValueError(f"unsupported rope_type {rope_type!r}")
    return inv_freq.to(torch.float32)


class RotaryEncoding(PositionEncoding):
    def __init__(self, *, rot_dim: int, theta: float, scaling: dict | None = None,
                 interleaved: bool = False) -> None:
        if rot_dim <= 0 or rot_dim % 2:
            raise ValueError(f"rotary dimension must be positive and even, got {rot_dim}")
        self.rot_dim = rot_dim
        self.theta = theta
        self.scaling = scaling
        self.interleaved = interleaved
        self._key = ("rotary", id(self))

    def setup(self, runtime) -> None:
        super().setup(runtime)
        self.inv_freq = rotary_inv_freq(self.rot_dim, self.theta, self.scaling).to(runtime.device)

    def prepare(self, ctx) -> None:
        half = self.rot_dim // 2
        cos = ctx.buf(f"rope_cos_{id(self)}", half, torch.float32)
        sin = ctx.buf(f"rope_sin_{id(self)}", half, torch.float32)
        ops.rope_table(cos, sin, ctx.positions, self.inv_freq)
        ctx.scratch[self._key] = RotaryTables(cos, sin, self.rot_dim, self.interleaved)

    def rotary(self, ctx) -> RotaryTables:
        return ctx.scratch[self._key]


class NoPositionEncoding(PositionEncoding):
    """Nothing is rotated and nothing is added."""


register_position_encoding("rotary", RotaryEncoding)
register_position_encoding("none", NoPositionEncoding)
