"""Token embedding and output head.

Reference: kvcore/model/models/llama3.py:161-165,178-180 (a plain gather; the padding
index has no effect on the forward pass) and :219-225,245-247 with
kvcore/sample/logits_processor.py:30-54 (no bias; with tied embeddings the head's
matrix is the embedding's).  Logits leave the head as float32.
"""

from __future__ import annotations

import torch

from kvcore_amd.ops import library as ops

from .base import ParamSpec, Part


class TokenEmbedding(Part):
    def __init__(self, *, vocab_size: int, hidden_size: int) -> None:
        self.vocab_size = vocab_size
        self.hidden_size = hidden_size

    def param_specs(self) -> list[ParamSpec]:
        return [ParamSpec("weight", (self.vocab_size, self.hidden_size))]

    def forward(self, residual: torch.Tensor, token_ids: torch.Tensor) -> None:
        ops.embed(residual, self.params["weight"], token_ids)


class OutputHead(Part):
    """``tied`` heads own no parameter; the model binds the embedding matrix to them."""

    def __init__(self, *, vocab_size: int, hidden_size: int, tied: bool) -> None:
        self.vocab_size = vocab_size
        self.hidden_size = hidden_size
        self.tied = tied

    def param_specs(self) -> list[ParamSpec]:
        return [] if self.tied else [ParamSpec("weight", (self.vocab_size, self.hidden_size))]

    def product_weights(self) -> tuple[str, ...]:
        return ("weight",)

    def forward(self, logits: torch.Tensor, hidden_rows: torch.Tensor, ctx) -> None:
        """``logits [S, V]`` float32 from ``hidden_rows [S, H]`` in the model dtype."""
        w = self.params["weight"]
        if hidden_rows.dtype == torch.float32:
            ops.linear(logits, hidden_rows, w)
            return
        S = hidden_rows.shape[0]
        # measured at 128256 x 4096: the few-row kernel wins up to 12 rows, the kernel that
        # shares the rows through LDS from 24 on (215 against 231 us at 64 rows), the vendor
        # product with a conversion afterwards in between and beyond 64
        if self.hidden_size % 8 == 0 and (S <= 12 or (S <= ops.SKINNY_PREFERRED_ROWS
                                                       and self.vocab_size < 65536)):
            ops.linear(logits, hidden_rows, w)  # float32 sums are stored without rounding
            return
        if ops.SKINNY_PREFERRED_ROWS < S <= ops.MID_ROWS and ops.mid_operands_ok(hidden_rows, w) \
                and logits.stride(1) == 1:
            ops.gemm_mid(logits, hidden_rows, w, mode=0)  # float32 sums, stored as they are
            return
        low = ctx.buffers.get("head_logits_dt", S, self.vocab_size, hidden_rows.dtype,
                              reserve=ctx.buffers.seq_capacity)
        ops.linear(low, hidden_rows, w)
        ops.to_float(logits, low)
