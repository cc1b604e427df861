"""Token embedding and output head.

Reference: kvcore/model/models/llama3.py:161-165,178-180 (a plain gather; the padding
index has no effect on the forward pass) and :219-225,245-247 with
kvcore/sample/logits_processor.py:30-54 (the product, an optional bias, an optional soft
cap ``cap * tanh(x / cap)``, then a scale; with tied embeddings the head's matrix is the
embedding's).  Logits leave the head as float32 sums, whatever the number of rows.
"""

from __future__ import annotations

import torch

from kvcore_amd.ops import library as ops

from .base import Embedding, Head, ParamSpec, register_embedding, register_head


class TokenEmbedding(Embedding):
    """``scale`` multiplies the embedded rows (1.0 for Llama; some architectures use
    ``sqrt(hidden_size)``)."""

    def __init__(self, *, vocab_size: int, hidden_size: int, scale: float = 1.0) -> None:
        self.vocab_size = vocab_size
        self.hidden_size = hidden_size
        self.scale = float(scale)

    def param_specs(self) -> list[ParamSpec]:
        return [ParamSpec("weight", (self.vocab_size, self.hidden_size))]

    def forward(self, residual: torch.Tensor, token_ids: torch.Tensor) -> None:
        ops.embed(residual, self.params["weight"], token_ids, self.scale)


class LinearHead(Head):
    """``logits = hidden @ W.T (+ bias)``, then ``soft_cap * tanh(logits / soft_cap)`` if
    ``soft_cap > 0``, then ``* logit_scale``.  ``tied`` heads own no matrix; the model binds
    the embedding matrix to them."""

    def __init__(self, *, vocab_size: int, hidden_size: int, tied: bool = False, bias: bool = False,
                 logit_scale: float = 1.0, soft_cap: float = 0.0) -> None:
        if soft_cap < 0:
            raise ValueError(f"soft_cap must be positive when set, got {soft_cap}")
        self.vocab_size = vocab_size
        self.hidden_size = hidden_size
        self.tied = tied
        self.bias = bias
        self.logit_scale = float(logit_scale)
        self.soft_cap = float(soft_cap)

    def param_specs(self) -> list[ParamSpec]:
        specs = [] if self.tied else [ParamSpec("weight", (self.vocab_size, self.hidden_size))]
        if self.bias:
            specs.append(ParamSpec("bias", (self.vocab_size,), init="zeros"))
        return specs

    def product_weights(self) -> tuple[str, ...]:
        return ("weight",)

    def forward(self, logits: torch.Tensor, hidden_rows: torch.Tensor, ctx) -> None:
        """``logits [S, V]`` float32 from ``hidden_rows [S, H]`` in the model dtype."""
        self._product(logits, hidden_rows)
        bias = self.params.get("bias")
        if bias is not None or self.soft_cap > 0 or self.logit_scale != 1.0:
            ops.logits_finish(logits, bias, self.soft_cap, self.logit_scale)

    def _product(self, logits: torch.Tensor, hidden_rows: torch.Tensor) -> None:
        """Every kernel that ``ops.linear`` may choose stores the float32 sums unrounded, so a
        request's logits do not change their rounding with the number of rows beside it."""
        ops.linear(logits, hidden_rows, self.params["weight"])


OutputHead = LinearHead

register_embedding("token_embedding", TokenEmbedding)
register_head("linear_head", LinearHead)
