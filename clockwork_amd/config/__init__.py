from clockwork_amd.config.engine import CacheConfig, EngineConfig, ModelConfig, SchedulerConfig
from clockwork_amd.config.spec import (
    LayerSpec,
    ModelSpec,
    RunEntry,
)

__all__ = [
    "CacheConfig",
    "EngineConfig",
    "ModelConfig",
    "SchedulerConfig",
    "LayerSpec",
    "ModelSpec",
    "RunEntry",
]
