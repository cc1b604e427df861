"""kvcore_amd: a small, whole LLM inference engine for one MI355X.

From a model folder (config.json + safetensors) to generated tokens: typed
configuration, architecture registry, weights by name, layers assembled from parts,
a paged KV cache manager, one step function for mixed batches, a scheduler with
chunked prefill, sampling, and hand-written gfx950 kernels underneath.
"""

from .config.engine_config import (  # noqa: F401
    CacheConfig, DeviceConfig, KVCoreConfig, LoadConfig, ModelConfig, SchedulerConfig,
)
from .sampling.params import SamplingParams  # noqa: F401

__all__ = [
    "CacheConfig", "DeviceConfig", "KVCoreConfig", "LoadConfig", "ModelConfig", "SchedulerConfig",
    "SamplingParams", "LLMEngine", "GenerationRequest", "GenerationOutput",
]


def __getattr__(name):
    if name in ("LLMEngine", "GenerationRequest", "GenerationOutput"):
        from .engine import llm_engine

        return getattr(llm_engine, name)
    raise AttributeError(name)
