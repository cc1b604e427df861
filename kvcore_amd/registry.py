"""One registry from an architecture's name to how its model is made.

The key is ``architectures[0]`` of config.json, with ``model_type`` as a second chance
(the reference keys on ``model_type`` alone: kvcore/model/model_loader/
default_loader.py:32-36,64-70).  An entry holds a parser from the raw config mapping to
a typed configuration and a function from that configuration to a ``ModelSpec``.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Callable, Mapping

from kvcore_amd.models.spec import ModelSpec


@dataclass(frozen=True)
class Architecture:
    name: str
    parse_config: Callable[[Mapping[str, Any]], Any]
    build_spec: Callable[[Any], ModelSpec]


MODEL_REGISTRY: dict[str, Architecture] = {}


def register_architecture(name: str, parse_config: Callable[[Mapping[str, Any]], Any],
                          build_spec: Callable[[Any], ModelSpec], *, aliases: tuple[str, ...] = (),
                          replace: bool = False) -> None:
    arch = Architecture(name, parse_config, build_spec)
    for key in (name, *aliases):
        if key in MODEL_REGISTRY and not replace:
            raise ValueError(f"architecture {key!r} is already registered")
        MODEL_REGISTRY[key] = arch


def unregister_architecture(name: str) -> None:
    MODEL_REGISTRY.pop(name, None)


def resolve_architecture(config: Mapping[str, Any]) -> Architecture:
    names = list(config.get("architectures") or [])
    if config.get("model_type"):
        names.append(config["model_type"])
    for name in names:
        if name in MODEL_REGISTRY:
            return MODEL_REGISTRY[name]
    raise ValueError(
        f"Unsupported architecture {names or None!r}. Supported: {sorted(MODEL_REGISTRY)}"
    )


def _register_builtin() -> None:
    from kvcore_amd.config.model_config import LlamaConfig
    from kvcore_amd.models.llama import llama_spec

    register_architecture("LlamaForCausalLM", LlamaConfig.from_dict, llama_spec, aliases=("llama",))


_register_builtin()
