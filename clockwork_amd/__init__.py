"""clockwork_amd: a single-GPU MI355X (gfx950) inference engine for dense Qwen2-style decoders.

Control (configuration, cache manager, scheduler, entry points) is Python; every
operation of the forward pass is a hand-written HIP kernel loaded from in-tree
shared libraries (see ``clockwork_amd.csrc``).
"""

__version__ = "0.1.0"

from clockwork_amd.config.engine import (  # noqa: F401
    CacheConfig,
    EngineConfig,
    ModelConfig,
    SchedulerConfig,
)
from clockwork_amd.engine.sequence import RequestOutput, SamplingParams  # noqa: F401


def __getattr__(name):
    # LLMEngine pulls in torch and the HIP libraries; import it on first use only.
    if name == "LLMEngine":
        from clockwork_amd.engine.llm_engine import LLMEngine

        return LLMEngine
    raise AttributeError(name)
