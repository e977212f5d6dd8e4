"""Per-request state shared by the scheduler, the cache manager and the engine.

Same fields and meanings as the reference (clockwork/engine/sequence.py:10-96);
block tables live in the cache manager, keyed by ``seq_id``, because a request
may hold one table per layer group.
"""

from __future__ import annotations

import time
from dataclasses import dataclass, field
from enum import Enum
from typing import Optional


class SequenceStatus(Enum):
    WAITING = "waiting"
    RUNNING = "running"
    PREEMPTED = "preempted"
    FINISHED_STOPPED = "finished_stopped"
    FINISHED_LENGTH = "finished_length"
    FINISHED_ABORTED = "finished_aborted"


_FINISHED = frozenset(
    {
        SequenceStatus.FINISHED_STOPPED,
        SequenceStatus.FINISHED_LENGTH,
        SequenceStatus.FINISHED_ABORTED,
    }
)


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


class Sequence:
    """Tokens of one request and how many of them have keys and values in the cache."""

    def __init__(
        self,
        seq_id: str,
        prompt_token_ids: list[int],
        sampling_params: Optional[SamplingParams] = None,
        arrival_time: Optional[float] = None,
    ) -> None:
        self.seq_id = seq_id
        self.prompt_token_ids = list(prompt_token_ids)
        self.output_token_ids: list[int] = []
        self.sampling_params = sampling_params if sampling_params is not None else SamplingParams()
        self.status = SequenceStatus.WAITING
        self.num_computed_tokens = 0
        self.num_cached_tokens = 0
        self.arrival_time = time.monotonic() if arrival_time is None else arrival_time

    def token_ids(self) -> list[int]:
        return self.prompt_token_ids + self.output_token_ids

    def tokens_in(self, start: int, end: int) -> list[int]:
        """Tokens at positions [start, end) without building the whole list."""
        n_prompt = len(self.prompt_token_ids)
        if end <= n_prompt:
            return self.prompt_token_ids[start:end]
        if start >= n_prompt:
            return self.output_token_ids[start - n_prompt : end - n_prompt]
        return self.prompt_token_ids[start:] + self.output_token_ids[: end - n_prompt]

    def __len__(self) -> int:
        return len(self.prompt_token_ids) + len(self.output_token_ids)

    def append_token(self, token_id: int) -> None:
        self.output_token_ids.append(int(token_id))

    def is_finished(self) -> bool:
        return self.status in _FINISHED

    def num_uncomputed_tokens(self) -> int:
        return len(self) - self.num_computed_tokens

    def is_prefilling(self) -> bool:
        """More than the last token still has to be run (a prompt, or a recompute after preemption)."""
        return self.num_uncomputed_tokens() > 1

    def reset_for_recompute(self) -> None:
        # clockwork/engine/sequence.py:79-82: progress is dropped, tokens are kept
        self.num_computed_tokens = 0

    def __repr__(self) -> str:
        return (
            f"Sequence({self.seq_id!r}, len={len(self)}, computed={self.num_computed_tokens}, "
            f"{self.status.value})"
        )


@dataclass
class RequestOutput:
    """clockwork/engine/sequence.py:85-96."""

    request_id: str
    prompt_token_ids: list[int]
    token_ids: list[int]
    text: str
    finished: bool
    finish_reason: Optional[str]
    num_cached_tokens: int
    num_prompt_tokens: int
    num_generated_tokens: int
    delta_text: str = ""
