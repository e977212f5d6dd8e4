"""What a request asks of the sampler and of the finish rules."""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Optional


@dataclass
class SamplingParams:
    """clockwork/engine/sequence.py:28-41. ``temperature == 0`` means greedy."""

    max_tokens: int = 64
    temperature: float = 0.0
    top_p: float = 1.0
    top_k: int = -1
    stop: list[str] = field(default_factory=list)
    stop_token_ids: list[int] = field(default_factory=list)
    ignore_eos: bool = False
    seed: Optional[int] = None

    @property
    def greedy(self) -> bool:
        return self.temperature == 0.0
