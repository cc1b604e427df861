"""Typed architecture configuration read from a model folder's ``config.json``.

Every size and constant of the model comes from the file.  A key the file must
carry raises a ``ConfigError`` that names it; optional keys take the defaults the
reference takes (cited per field).
"""

from __future__ import annotations

import json
from dataclasses import dataclass, field
from pathlib import Path
from typing import Any, Mapping


class ConfigError(ValueError):
    """config.json is missing a key, or holds a value this engine refuses."""


def _require(d: Mapping[str, Any], key: str, kind: type) -> Any:
    if key not in d or d[key] is None:
        raise ConfigError(f"config.json: missing required key {key!r}")
    value = d[key]
    if kind is int and (isinstance(value, bool) or not isinstance(value, int)):
        raise ConfigError(f"config.json: {key!r} must be an integer, got {value!r}")
    if kind is float and (isinstance(value, bool) or not isinstance(value, (int, float))):
        raise ConfigError(f"config.json: {key!r} must be a number, got {value!r}")
    return kind(value)


@dataclass(frozen=True)
class RopeScaling:
    """``rope_scaling`` of config.json.  ``rope_type`` is ``"default"`` (identity) or
    ``"llama3"``; any other type is refused.  The reference has no rope scaling
    (kvcore/model/layer/rotary_embedding.py:52-70 reads the base only)."""

    rope_type: str = "default"
    factor: float = 1.0
    low_freq_factor: float = 1.0
    high_freq_factor: float = 1.0
    original_max_position_embeddings: int = 0

    @classmethod
    def from_dict(cls, d: Mapping[str, Any] | None) -> "RopeScaling":
        if not d:
            return cls()
        rope_type = d.get("rope_type", d.get("type", "default")) or "default"
        if rope_type == "default":
            return cls()
        if rope_type != "llama3":
            raise ConfigError(
                f"config.json: rope_scaling.rope_type {rope_type!r} is not supported "
                "(supported: 'default', 'llama3')"
            )
        scaling = cls(
            rope_type="llama3",
            factor=_require(d, "factor", float),
            low_freq_factor=_require(d, "low_freq_factor", float),
            high_freq_factor=_require(d, "high_freq_factor", float),
            original_max_position_embeddings=_require(d, "original_max_position_embeddings", int),
        )
        if scaling.factor <= 0 or scaling.original_max_position_embeddings <= 0:
            raise ConfigError("config.json: rope_scaling factor and original length must be positive")
        if scaling.high_freq_factor <= scaling.low_freq_factor:
            raise ConfigError("config.json: rope_scaling.high_freq_factor must exceed low_freq_factor")
        return scaling

    def to_dict(self) -> dict[str, Any] | None:
        if self.rope_type == "default":
            return None
        return {
            "rope_type": self.rope_type,
            "factor": self.factor,
            "low_freq_factor": self.low_freq_factor,
            "high_freq_factor": self.high_freq_factor,
            "original_max_position_embeddings": self.original_max_position_embeddings,
        }


@dataclass(frozen=True)
class LlamaConfig:
    """The Llama 3 dense decoder's keys (reference: kvcore/model/models/llama3.py reads
    them from the Hugging Face config object at :26-38, :55-69, :161-176, :219-225)."""

    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    rms_norm_eps: float
    max_position_embeddings: int
    # default: the head count (kvcore/engine/engine_core.py:164)
    num_key_value_heads: int = 0
    # default: hidden_size // num_attention_heads (llama3.py:59)
    head_dim: int = 0
    # default 10000.0 (rotary_embedding.py:38-49)
    rope_theta: float = 10000.0
    rope_scaling: RopeScaling = field(default_factory=RopeScaling)
    tie_word_embeddings: bool = False
    attention_bias: bool = False  # llama3.py:61
    mlp_bias: bool = False  # llama3.py:32
    hidden_act: str = "silu"  # llama3.py:28-31 refuses anything else
    pad_token_id: int | None = None
    eos_token_ids: tuple[int, ...] = ()  # engine_core.py:209-217: an int or a list
    bos_token_id: int | None = None
    dtype: str | None = None  # model_loader/utils.py:10-16
    architectures: tuple[str, ...] = ("LlamaForCausalLM",)
    model_type: str = "llama"

    def __post_init__(self) -> None:
        if self.num_key_value_heads == 0:
            object.__setattr__(self, "num_key_value_heads", self.num_attention_heads)
        if self.head_dim == 0:
            if self.hidden_size % self.num_attention_heads:
                raise ConfigError(
                    "config.json: hidden_size is not a multiple of num_attention_heads "
                    "and no head_dim is given"
                )
            object.__setattr__(self, "head_dim", self.hidden_size // self.num_attention_heads)
        for name in (
            "vocab_size", "hidden_size", "intermediate_size", "num_hidden_layers",
            "num_attention_heads", "num_key_value_heads", "head_dim", "max_position_embeddings",
        ):
            if getattr(self, name) <= 0:
                raise ConfigError(f"config.json: {name} must be positive, got {getattr(self, name)}")
        if self.num_attention_heads % self.num_key_value_heads:
            raise ConfigError(
                f"config.json: num_attention_heads ({self.num_attention_heads}) is not a multiple "
                f"of num_key_value_heads ({self.num_key_value_heads})"
            )
        if self.head_dim % 2:
            raise ConfigError(f"config.json: head_dim must be even for rotary pairs, got {self.head_dim}")
        if self.rms_norm_eps <= 0:
            raise ConfigError(f"config.json: rms_norm_eps must be positive, got {self.rms_norm_eps}")
        if self.hidden_act != "silu":
            raise ConfigError(
                f"config.json: unsupported activation {self.hidden_act!r}; only 'silu' is supported"
            )

    @classmethod
    def from_dict(cls, d: Mapping[str, Any]) -> "LlamaConfig":
        rope_params = d.get("rope_parameters") or {}
        theta = rope_params.get("rope_theta", rope_params.get("theta", d.get("rope_theta")))
        scaling = d.get("rope_scaling")
        if scaling is None and rope_params.get("rope_type", "default") not in (None, "default"):
            scaling = rope_params
        eos = d.get("eos_token_id")
        if eos is None:
            eos_ids: tuple[int, ...] = ()
        elif isinstance(eos, (list, tuple)):
            eos_ids = tuple(int(e) for e in eos)
        else:
            eos_ids = (int(eos),)
        dtype = d.get("dtype", d.get("torch_dtype"))
        return cls(
            vocab_size=_require(d, "vocab_size", int),
            hidden_size=_require(d, "hidden_size", int),
            intermediate_size=_require(d, "intermediate_size", int),
            num_hidden_layers=_require(d, "num_hidden_layers", int),
            num_attention_heads=_require(d, "num_attention_heads", int),
            rms_norm_eps=_require(d, "rms_norm_eps", float),
            max_position_embeddings=_require(d, "max_position_embeddings", int),
            num_key_value_heads=int(d.get("num_key_value_heads") or 0),
            head_dim=int(d.get("head_dim") or 0),
            rope_theta=10000.0 if theta is None else float(theta),
            rope_scaling=RopeScaling.from_dict(scaling),
            tie_word_embeddings=bool(d.get("tie_word_embeddings", False)),
            attention_bias=bool(d.get("attention_bias", False)),
            mlp_bias=bool(d.get("mlp_bias", False)),
            hidden_act=str(d.get("hidden_act", "silu")),
            pad_token_id=d.get("pad_token_id"),
            eos_token_ids=eos_ids,
            bos_token_id=d.get("bos_token_id"),
            dtype=None if dtype is None else str(dtype).replace("torch.", ""),
            architectures=tuple(d.get("architectures") or ("LlamaForCausalLM",)),
            model_type=str(d.get("model_type", "llama")),
        )

    def to_dict(self) -> dict[str, Any]:
        out: dict[str, Any] = {
            "architectures": list(self.architectures),
            "model_type": self.model_type,
            "vocab_size": self.vocab_size,
            "hidden_size": self.hidden_size,
            "intermediate_size": self.intermediate_size,
            "num_hidden_layers": self.num_hidden_layers,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads,
            "head_dim": self.head_dim,
            "rms_norm_eps": self.rms_norm_eps,
            "max_position_embeddings": self.max_position_embeddings,
            "rope_theta": self.rope_theta,
            "rope_scaling": self.rope_scaling.to_dict(),
            "tie_word_embeddings": self.tie_word_embeddings,
            "attention_bias": self.attention_bias,
            "mlp_bias": self.mlp_bias,
            "hidden_act": self.hidden_act,
        }
        if self.pad_token_id is not None:
            out["pad_token_id"] = self.pad_token_id
        if self.bos_token_id is not None:
            out["bos_token_id"] = self.bos_token_id
        if self.eos_token_ids:
            out["eos_token_id"] = (
                self.eos_token_ids[0] if len(self.eos_token_ids) == 1 else list(self.eos_token_ids)
            )
        if self.dtype is not None:
            out["dtype"] = self.dtype
        return out


def read_generation_eos(model_dir: str | Path) -> tuple[int, ...]:
    """``eos_token_id`` (an int or a list) of ``<model_dir>/generation_config.json``; empty if
    the file or the key is absent.  Instruct checkpoints of Llama 3 list their end-of-turn
    id there and not in config.json."""
    path = Path(model_dir).expanduser() / "generation_config.json"
    if not path.is_file():
        return ()
    try:
        data = json.loads(path.read_text())
    except (OSError, ValueError) as exc:
        raise ConfigError(f"{path}: not readable as JSON: {exc}") from exc
    eos = data.get("eos_token_id") if isinstance(data, dict) else None
    if eos is None:
        return ()
    if isinstance(eos, (list, tuple)):
        return tuple(int(e) for e in eos)
    return (int(eos),)


def read_config_json(model_dir: str | Path) -> dict[str, Any]:
    """The raw mapping of ``<model_dir>/config.json``.  A missing folder raises
    ``FileNotFoundError`` as the reference does (model_loader/default_loader.py:98-102)."""
    folder = Path(model_dir).expanduser()
    if not folder.is_dir():
        raise FileNotFoundError(f"Model path does not exist: {folder}")
    path = folder / "config.json"
    if not path.is_file():
        raise FileNotFoundError(f"No config.json in model folder: {folder}")
    with open(path, "r", encoding="utf-8") as f:
        data = json.load(f)
    if not isinstance(data, dict):
        raise ConfigError(f"{path}: top level must be an object")
    return data
