"""Arrangements of norms, mixer and feed-forward around the residual stream.

Reference: kvcore/model/models/llama3.py:124-142.  The reference carries
``(hidden, residual)`` and lets each norm add the pending ``hidden`` first; this is
the same arrangement with the pending output called ``delta`` and the stream kept in
float32.
"""

from __future__ import annotations

import torch

from .base import Block, FeedForward, Mixer, Norm, Part, register_block


class PreNormBlock(Block):
    """``r += delta; a = mixer(norm_in(r)); r += a; out = ffn(norm_post(r))``, the last
    sum left pending for the next block's first norm."""

    NORM_NAMES = ("input_layernorm", "post_attention_layernorm")

    def __init__(self, *, mixer: Mixer, ffn: FeedForward, norms: dict[str, Norm],
                 mixer_name: str = "self_attn", ffn_name: str = "mlp") -> None:
        super().__init__(mixer=mixer, ffn=ffn, norms=norms)
        missing = [n for n in self.NORM_NAMES if n not in norms]
        if missing:
            raise ValueError(f"pre-norm block needs norms {self.NORM_NAMES}, missing {missing}")
        self.mixer_name = mixer_name
        self.ffn_name = ffn_name

    def children(self) -> dict[str, Part]:
        return {
            self.NORM_NAMES[0]: self.norms[self.NORM_NAMES[0]],
            self.mixer_name: self.mixer,
            self.NORM_NAMES[1]: self.norms[self.NORM_NAMES[1]],
            self.ffn_name: self.ffn,
        }

    def forward(self, delta: torch.Tensor | None, residual: torch.Tensor, ctx, call) -> torch.Tensor:
        x = ctx.buf("block_x", residual.shape[1])
        self.norms[self.NORM_NAMES[0]].forward_fused(x, residual, delta)
        a = self.mixer.forward(x, ctx, call)
        self.norms[self.NORM_NAMES[1]].forward_fused(x, residual, a)
        return self.ffn.forward(x, ctx, call)


register_block("prenorm", PreNormBlock)
