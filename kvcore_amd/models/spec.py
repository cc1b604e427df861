"""A model as data: layers chosen part by part, and the order in which they run."""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any

from kvcore_amd.parts.base import PartSpec


@dataclass(frozen=True)
class LayerSpec:
    """One layer's parts.  ``position`` indexes ``ModelSpec.positions`` (None: the mixer
    gets no position encoding); ``norms`` maps the block's norm names to norm specs;
    ``prefix`` is the layer's checkpoint prefix."""

    prefix: str
    mixer: PartSpec
    ffn: PartSpec
    norms: dict[str, PartSpec]
    block: PartSpec = field(default_factory=lambda: PartSpec("prenorm"))
    position: int | None = None


@dataclass(frozen=True)
class ScheduleEntry:
    """Run ``layer``.  ``cache_from`` names an earlier schedule entry (by its index in the
    schedule) whose cache this entry reads instead of writing its own."""

    layer: int
    cache_from: int | None = None


@dataclass(frozen=True)
class ModelSpec:
    vocab_size: int
    hidden_size: int
    max_position_embeddings: int
    layers: tuple[LayerSpec, ...]
    final_norm: PartSpec
    positions: tuple[PartSpec, ...] = ()
    schedule: tuple[ScheduleEntry, ...] = ()
    tie_word_embeddings: bool = False
    # the embedding and the head, chosen by kind like every other part; None stands for the
    # plain token embedding and the linear head (tied as ``tie_word_embeddings`` says) of
    # this vocabulary and width
    embedding: PartSpec | None = None
    head: PartSpec | None = None
    eos_token_ids: tuple[int, ...] = ()
    # checkpoint prefixes of the position encodings' own parameters, one per entry of
    # ``positions`` (empty: "model.positions.<i>"; a rotary encoding has no parameters)
    position_prefixes: tuple[str, ...] = ()
    embed_prefix: str = "model.embed_tokens"
    final_norm_prefix: str = "model.norm"
    head_prefix: str = "lm_head"
    # checkpoint names that may be present and are not read (reference:
    # kvcore/model/model_utils.py:49-50 skips rotary_emb.inv_freq buffers)
    ignored_suffixes: tuple[str, ...] = ("rotary_emb.inv_freq",)
    extra: dict[str, Any] = field(default_factory=dict)

    def resolved_schedule(self) -> tuple[ScheduleEntry, ...]:
        return self.schedule or tuple(ScheduleEntry(i) for i in range(len(self.layers)))

    def resolved_embedding(self) -> PartSpec:
        return self.embedding or PartSpec("token_embedding", {
            "vocab_size": self.vocab_size, "hidden_size": self.hidden_size})

    def resolved_head(self) -> PartSpec:
        return self.head or PartSpec("linear_head", {
            "vocab_size": self.vocab_size, "hidden_size": self.hidden_size,
            "tied": self.tie_word_embeddings})
