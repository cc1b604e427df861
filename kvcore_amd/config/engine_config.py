"""Engine configuration: frozen, validated sub-configs composed in ``KVCoreConfig``.

Names and meanings follow the reference's kvcore/config.py:15-192 where it has them;
sparse-KV and prefix-cache settings have no counterpart here.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from pathlib import Path

DTYPE_NAMES = {
    "bfloat16": "bfloat16",
    "bf16": "bfloat16",
    "float32": "float32",
    "fp32": "float32",
    "float": "float32",
}


# The reference chooses between "torch_paged" and "triton_paged" (config.py:28, 170-178);
# here the paged attention is always the HIP kernels.
ATTN_BACKENDS = ("hip",)


def canonical_dtype(name: str | None) -> str | None:
    """``"bfloat16"`` or ``"float32"`` from any of their usual spellings."""
    if name is None:
        return None
    key = str(name).replace("torch.", "").lower()
    if key not in DTYPE_NAMES:
        raise ValueError(f"unsupported dtype {name!r}; supported: bfloat16, float32")
    return DTYPE_NAMES[key]


@dataclass(frozen=True)
class ModelConfig:
    """Reference: config.py:15-30.  ``dtype`` None means: config.json's ``dtype`` if it
    is one of ours, else bfloat16."""

    model: str | Path
    tokenizer: str | Path | None = None
    dtype: str | None = None
    max_model_len: int | None = None
    attn_backend: str | None = None

    def __post_init__(self) -> None:
        if self.max_model_len is not None and self.max_model_len <= 0:
            raise ValueError(f"max_model_len must be positive, got {self.max_model_len}")
        if self.attn_backend not in (None, *ATTN_BACKENDS):
            raise ValueError(
                f"unsupported attn_backend {self.attn_backend!r}; this engine has one attention "
                f"backend: {', '.join(ATTN_BACKENDS)} (the HIP kernels for gfx950)")
        object.__setattr__(self, "dtype", canonical_dtype(self.dtype))


@dataclass(frozen=True)
class LoadConfig:
    """Reference: config.py:33-40.  ``load_format`` is ``"safetensors"`` (read the
    folder's files) or ``"random"`` (fill every parameter from ``seed``; the folder
    then needs only config.json).  ``strict`` also refuses unexpected tensors, which
    the reference drops silently (kvcore/model/model_utils.py:65-76).
    ``pack_decode_weights``: keep a second copy of the bfloat16 weight matrices in the order
    in which decode steps of few tokens stream them (``ops.pack_weight``: some 6% off such a
    step for twice the weights' memory); None decides by the room on the device."""

    load_format: str = "safetensors"
    strict: bool = True
    seed: int = 0
    pack_decode_weights: bool | None = None

    def __post_init__(self) -> None:
        if self.load_format not in ("safetensors", "random", "auto"):
            raise ValueError(f"load_format must be 'safetensors' or 'random', got {self.load_format!r}")


@dataclass(frozen=True)
class CacheConfig:
    """Reference: config.py:43-60.  ``num_gpu_blocks`` counts pages including the
    reserved null page; when given it wins over profiling.  ``poison_pages`` is a debugging
    aid of this engine: every page is filled with NaN when a request first gets it and when
    it is given back, so that a read of a slot its request did not write shows in the logits
    (the reference zeroes new blocks instead, kvcore/model/model_runner.py:646-657)."""

    block_size: int = 16
    num_gpu_blocks: int | None = None
    profile_kv_cache: bool = True
    gpu_memory_utilization: float = 0.9
    poison_pages: bool = False

    def __post_init__(self) -> None:
        if self.block_size <= 0:
            raise ValueError(f"block_size must be positive, got {self.block_size}")
        if self.num_gpu_blocks is not None and self.num_gpu_blocks <= 1:
            raise ValueError(f"num_gpu_blocks must exceed 1 (page 0 is reserved), got {self.num_gpu_blocks}")
        if not 0 < self.gpu_memory_utilization <= 1:
            raise ValueError(
                f"gpu_memory_utilization must be in (0, 1], got {self.gpu_memory_utilization}"
            )


@dataclass(frozen=True)
class SchedulerConfig:
    """Reference: config.py:63-93 (same five names, same validation).
    ``max_num_partial_prefills`` left unset means ``max_num_seqs``: every request that fits
    may be in its prompt at once (the reference's own default is 1, and its command line
    raises it to 128: scripts/run_llm_engine_offline_batch.py:145).  ``decode_run_ahead``
    is this engine's own: while requests only decode, the next step is launched before the
    tokens of the step in flight have reached the host (``Scheduler.plan_decode_ahead``)."""

    max_num_seqs: int = 8
    max_num_scheduled_tokens: int = 512
    max_num_partial_prefills: int | None = None
    max_long_partial_prefills: int = 1
    long_prefill_token_threshold: int = 0
    decode_run_ahead: bool = True

    def __post_init__(self) -> None:
        if self.max_num_partial_prefills is None:
            object.__setattr__(self, "max_num_partial_prefills", self.max_num_seqs)
        for name in (
            "max_num_seqs", "max_num_scheduled_tokens",
            "max_num_partial_prefills", "max_long_partial_prefills",
        ):
            if getattr(self, name) <= 0:
                raise ValueError(f"{name} must be positive, got {getattr(self, name)}")
        if self.long_prefill_token_threshold < 0:
            raise ValueError(
                f"long_prefill_token_threshold must be non-negative, got {self.long_prefill_token_threshold}"
            )


@dataclass(frozen=True)
class DeviceConfig:
    """Reference: config.py:160-162.  ROCm torch names HIP devices ``cuda``."""

    device: str = "cuda:0"
    use_hip_graphs: bool = True


@dataclass(frozen=True)
class KVCoreConfig:
    """Reference: config.py:165-192."""

    model_config: ModelConfig
    load_config: LoadConfig = field(default_factory=LoadConfig)
    cache_config: CacheConfig = field(default_factory=CacheConfig)
    scheduler_config: SchedulerConfig = field(default_factory=SchedulerConfig)
    device_config: DeviceConfig = field(default_factory=DeviceConfig)

    def __post_init__(self) -> None:
        # an unset attention backend is filled in, as the reference does (config.py:170-192)
        if self.model_config.attn_backend is None:
            object.__setattr__(self.model_config, "attn_backend", ATTN_BACKENDS[0])
