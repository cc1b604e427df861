"""Arrangements of norms, mixer and feed-forward around the residual stream.

Reference: kvcore/model/models/llama3.py:124-142.  The reference carries
``(hidden, residual)`` and lets each norm add the pending ``hidden`` first; this is
the same arrangement with the pending output called ``delta`` and the stream kept in
float32.
"""

from __future__ import annotations

import torch

from kvcore_amd.ops import library as ops

from .base import Block, FeedForward, Mixer, Norm, Part, register_block


class PreNormBlock(Block):
    """``r += delta; a = mixer(norm_in(r)); r += a; out = ffn(norm_post(r))``, the last
    sum left pending for the next block's first norm."""

    def __init__(self, *, mixer: Mixer, ffn: FeedForward, norms: dict[str, Norm],
                 mixer_name: str = "self_attn", ffn_name: str = "mlp",
                 input_norm: str | None = None, post_norm: str | None = None) -> None:
        """``input_norm`` and ``post_norm`` name the norm before the mixer and the norm before
        the feed-forward among ``norms`` (they are also the norms' checkpoint sub-prefixes);
        left out, they are the first and the second norm that the layer lists."""
        super().__init__(mixer=mixer, ffn=ffn, norms=norms)
        listed = list(norms)
        if input_norm is None and listed:
            input_norm = listed[0]
        if post_norm is None:
            post_norm = next((n for n in listed if n != input_norm), None)
        missing = [n for n in (input_norm, post_norm) if n not in norms]
        if missing or input_norm == post_norm:
            raise ValueError(f"a pre-norm block needs two norms, one before the mixer and one before the "
                             f"feed-forward; asked for {(input_norm, post_norm)}, given {listed}")
        self.norm_names = (input_norm, post_norm)
        self.mixer_name = mixer_name
        self.ffn_name = ffn_name

    def children(self) -> dict[str, Part]:
        return {
            self.norm_names[0]: self.norms[self.norm_names[0]],
            self.mixer_name: self.mixer,
            self.norm_names[1]: self.norms[self.norm_names[1]],
            self.ffn_name: self.ffn,
        }

    def input_gain(self, scaled: bool = True):
        """The first norm as (gain, eps) if the block before may do its work: leaving scaled
        rows for this block's mixer to finish (``scaled``), or finishing it itself."""
        gain = self.norms[self.norm_names[0]].as_gain()
        if scaled and not self.mixer.takes_scaled_rows:
            return None
        return gain

    def forward(self, delta, residual: torch.Tensor, ctx, call, next_block=None):
        # With very few rows of bfloat16 the norms fold into the products around them: the product
        # before a norm adds into the residual and keeps the sums of squares, the product after
        # it applies the scale factor.  Otherwise every norm is a kernel of its own.
        # With a few dozen rows the product before a norm leaves partial sums of slices along
        # K, and one kernel adds them into the residual and normalises.
        fold, sums = self.norm_folding(ctx, residual.shape[1])
        if isinstance(delta, ops.ScaledRows):
            x = delta  # the block before made the first norm's rows
        elif isinstance(delta, ops.NormedRows):
            x = delta.data  # the block before did the first norm
        else:
            x = ctx.buf("block_x", residual.shape[1])
            self.norms[self.norm_names[0]].forward_fused(x, residual, delta)

        post = self.norms[self.norm_names[1]]
        gain = None
        if self.mixer.takes_sink and ((fold and self.ffn.takes_scaled_rows) or sums):
            gain = post.as_gain()
        if gain is not None:
            x2 = self.mixer.forward(x, ctx, call, sink=self.residual_sink(ctx, residual, gain, "block_x2", fold))
            if isinstance(x2, ops.NormedRows):
                x2 = x2.data
        else:
            a = self.mixer.forward(x, ctx, call)
            x2 = ctx.buf("block_x2", residual.shape[1])
            post.forward_fused(x2, residual, a)

        gain = None
        if next_block is not None and self.ffn.takes_sink and (fold or sums):
            gain = next_block.input_gain(scaled=fold)
        if gain is not None:
            return self.ffn.forward(x2, ctx, call, sink=self.residual_sink(ctx, residual, gain, "block_x", fold))
        return self.ffn.forward(x2, ctx, call)


register_block("prenorm", PreNormBlock)
