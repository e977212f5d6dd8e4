"""Two registries: architecture name -> how to build it, and part spec type -> implementation.

Both are open: a test or a user module registers a new mixer, feed-forward,
norm, position encoding, block arrangement or whole architecture without
touching the framework's files.
"""

from __future__ import annotations

import importlib
from dataclasses import dataclass
from typing import Any, Callable

from clockwork_amd.config.spec import ModelSpec, WeightTarget


@dataclass(frozen=True)
class Architecture:
    """What the engine needs to know about one architecture.

    ``parse_config(dict) -> cfg`` reads ``config.json`` keys into a typed object
    and rejects what is not built; ``build_spec(cfg) -> ModelSpec`` chooses the
    parts layer by layer; ``weight_plan(cfg, spec) -> list[WeightTarget]`` maps
    checkpoint tensor names onto the model's parameters.
    """

    name: str
    parse_config: Callable[[dict], Any]
    build_spec: Callable[[Any], ModelSpec]
    weight_plan: Callable[[Any, ModelSpec], list[WeightTarget]]


_ARCHITECTURES: dict[str, Architecture] = {}
_BUILTIN_ARCHITECTURES = {
    "Qwen2ForCausalLM": "clockwork_amd.models.qwen2",
    "qwen2": "clockwork_amd.models.qwen2",
}


def register_architecture(names: list[str], arch: Architecture) -> None:
    for name in names:
        _ARCHITECTURES[name] = arch


def unregister_architecture(names: list[str]) -> None:
    for name in names:
        _ARCHITECTURES.pop(name, None)


def resolve_architecture(config: dict) -> Architecture:
    """Pick the architecture by ``architectures[0]``, else by ``model_type``.

    Anything unknown is refused (the reference refuses every model_type but its own,
    clockwork/engine/loader.py:70-71; an architecture's ``parse_config`` repeats that check
    for its own name).
    """
    keys = []
    archs = config.get("architectures")
    if isinstance(archs, (list, tuple)) and archs:
        keys.append(archs[0])
    if config.get("model_type") is not None:
        keys.append(config["model_type"])
    for key in keys:
        if key not in _ARCHITECTURES and key in _BUILTIN_ARCHITECTURES:
            importlib.import_module(_BUILTIN_ARCHITECTURES[key])
        if key in _ARCHITECTURES:
            return _ARCHITECTURES[key]
    known = sorted(set(_ARCHITECTURES) | set(_BUILTIN_ARCHITECTURES))
    raise ValueError(
        f"no architecture is registered for model_type={config.get('model_type')!r} "
        f"architectures={config.get('architectures')!r}; registered: {known}"
    )


# ---- parts -------------------------------------------------------------------------------

# spec type -> factory(spec) -> part object. Built-in kinds are imported lazily so
# that registering and resolving specs needs neither torch nor the HIP libraries.
_PART_FACTORIES: dict[type, Callable[[Any], Any]] = {}
_BUILTIN_PARTS = {
    "RMSNormSpec": ("clockwork_amd.parts.norm", "RMSNorm"),
    "RopeNeoxSpec": ("clockwork_amd.parts.rope", "RopeNeox"),
    "AttentionSpec": ("clockwork_amd.parts.attention", "PagedAttention"),
    "SwiGLUSpec": ("clockwork_amd.parts.mlp", "SwiGLU"),
    "TokenEmbeddingSpec": ("clockwork_amd.parts.embedding", "TokenEmbedding"),
    "LinearHeadSpec": ("clockwork_amd.parts.embedding", "LinearHead"),
}
_ARRANGEMENTS: dict[str, Callable[..., Any]] = {}
_BUILTIN_ARRANGEMENTS = {"prenorm": ("clockwork_amd.parts.block", "PreNormBlock")}


def register_part(spec_type: type, factory: Callable[[Any], Any]) -> None:
    """Make ``factory(spec)`` the implementation of every spec of ``spec_type``."""
    _PART_FACTORIES[spec_type] = factory


def unregister_part(spec_type: type) -> None:
    _PART_FACTORIES.pop(spec_type, None)


def build_part(spec: Any) -> Any:
    factory = _PART_FACTORIES.get(type(spec))
    if factory is None:
        builtin = _BUILTIN_PARTS.get(type(spec).__name__)
        if builtin is None or type(spec).__module__ != "clockwork_amd.parts.specs":
            raise KeyError(f"no part is registered for spec type {type(spec).__name__}")
        factory = getattr(importlib.import_module(builtin[0]), builtin[1])
        _PART_FACTORIES[type(spec)] = factory
    return factory(spec)


def register_arrangement(name: str, factory: Callable[..., Any]) -> None:
    _ARRANGEMENTS[name] = factory


def unregister_arrangement(name: str) -> None:
    _ARRANGEMENTS.pop(name, None)


def build_arrangement(name: str, **parts) -> Any:
    factory = _ARRANGEMENTS.get(name)
    if factory is None:
        builtin = _BUILTIN_ARRANGEMENTS.get(name)
        if builtin is None:
            raise KeyError(f"no block arrangement named {name!r} is registered")
        factory = getattr(importlib.import_module(builtin[0]), builtin[1])
        _ARRANGEMENTS[name] = factory
    return factory(**parts)
