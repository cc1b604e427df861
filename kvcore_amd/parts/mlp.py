"""Gated feed-forward: ``down(silu(gate(x)) * up(x))`` with gate and up stacked.

Reference: kvcore/model/models/llama3.py:25-45 (gate rows first, then up rows) and
kvcore/model/layer/activation.py:14-16.
"""

from __future__ import annotations

import torch

from kvcore_amd.ops import library as ops

from .base import FeedForward, ParamSource, ParamSpec, register_feed_forward


class SwiGLU(FeedForward):
    @property
    def takes_scaled_rows(self) -> bool:  # x only goes into the gate-up product
        return self.hidden_size % 8 == 0

    @property
    def takes_sink(self) -> bool:
        return self.intermediate_size % 8 == 0

    def __init__(self, *, hidden_size: int, intermediate_size: int, bias: bool = False) -> None:
        self.hidden_size = hidden_size
        self.intermediate_size = intermediate_size
        self.bias = bias

    def param_specs(self) -> list[ParamSpec]:
        I, H = self.intermediate_size, self.hidden_size

        def stacked(suffix: str) -> tuple[ParamSource, ...]:
            return (ParamSource(f"gate_proj.{suffix}", 0, I), ParamSource(f"up_proj.{suffix}", I, I))

        specs = [
            ParamSpec("gate_up_proj.weight", (2 * I, H), sources=stacked("weight")),
            ParamSpec("down_proj.weight", (H, I)),
        ]
        if self.bias:
            specs.append(ParamSpec("gate_up_proj.bias", (2 * I,), init="zeros", sources=stacked("bias")))
            specs.append(ParamSpec("down_proj.bias", (H,), init="zeros"))
        return specs

    def product_weights(self) -> tuple[str, ...]:
        return ("gate_up_proj.weight", "down_proj.weight")

    def forward(self, x, ctx, call, sink=None):
        p = self.params
        act = ctx.buf("ffn_act", self.intermediate_size)
        # few rows: the product and the activation are one kernel and gate_up is never stored
        ops.linear_silu_mul(act, x, p["gate_up_proj.weight"], p.get("gate_up_proj.bias"),
                            lambda: ctx.buf("ffn_gate_up", 2 * self.intermediate_size))
        if sink is not None:
            return ops.linear(sink, act, p["down_proj.weight"], p.get("down_proj.bias"))
        out = ctx.buf("ffn_out", self.hidden_size)
        ops.linear(out, act, p["down_proj.weight"], p.get("down_proj.bias"))
        return out


register_feed_forward("swiglu", SwiGLU)
