"""Per-request state shared by the scheduler, the cache manager and the engine.

Same fields and meanings as the reference (clockwork/engine/sequence.py:10-82);
block tables live in the cache manager, keyed by ``seq_id``, because a request
may hold one table per layer group. ``SamplingParams`` (sampling/params.py) and
``RequestOutput`` (engine/outputs.py) can be imported from here as in the reference.
"""

from __future__ import annotations

import time
from enum import Enum
from typing import Optional

from clockwork_amd.engine.outputs import RequestOutput  # noqa: F401  (the reference keeps it in this module)
from clockwork_amd.sampling.params import SamplingParams


class SequenceStatus(Enum):
    WAITING = "waiting"
    RUNNING = "running"
    PREEMPTED = "preempted"
    FINISHED_STOPPED = "finished_stopped"
    FINISHED_LENGTH = "finished_length"
    FINISHED_ABORTED = "finished_aborted"


# the three ways a request ends (stop token or string, length, abort)
_FINISHED = frozenset(status for status in SequenceStatus if status.name.startswith("FINISHED_"))


class Sequence:
    """One request as the scheduler and the engine see it: its tokens, how far the cache has
    followed them, and where it stands (the fields of clockwork/engine/sequence.py:44-82, without
    the block table).

    The engine runs a request in portions, so its progress is a position: tokens before
    ``num_computed_tokens`` have their keys and values in the cache (``num_cached_tokens`` of them
    came from the prefix cache at admission), the tokens from there to the end are still to run.
    A request whose last token alone is to run is decoding; one with more is prefilling, whether
    that is a fresh prompt or a recompute after it was preempted."""

    __slots__ = ("seq_id", "prompt_token_ids", "output_token_ids", "sampling_params", "status",
                 "num_computed_tokens", "num_cached_tokens", "arrival_time")

    def __init__(self, seq_id: str, prompt_token_ids: list[int], sampling_params: Optional[SamplingParams] = None,
                 arrival_time: Optional[float] = None) -> None:
        self.seq_id = seq_id
        # plain ints (a list of them is taken as it is: an engine's prompt may be tens of thousands long)
        plain = type(prompt_token_ids) is list and set(map(type, prompt_token_ids)) <= {int}
        self.prompt_token_ids = list(prompt_token_ids) if plain else [int(t) for t in prompt_token_ids]
        self.output_token_ids: list[int] = []
        self.sampling_params = sampling_params or SamplingParams()
        self.arrival_time = arrival_time if arrival_time is not None else time.monotonic()
        self.status = SequenceStatus.WAITING
        self.num_cached_tokens = 0
        self.num_computed_tokens = 0

    # ------------------------------------------------------------------ tokens
    def __len__(self) -> int:
        return len(self.prompt_token_ids) + len(self.output_token_ids)

    def token_ids(self) -> list[int]:
        return [*self.prompt_token_ids, *self.output_token_ids]

    def tokens_in(self, start: int, end: int) -> list[int]:
        """The tokens at positions [start, end): a portion's input, cut from whichever of the two
        lists holds it (the whole sequence is not put together for it)."""
        boundary = len(self.prompt_token_ids)
        head = self.prompt_token_ids[start:end] if start < boundary else []
        if end <= boundary:
            return head
        return head + self.output_token_ids[max(start - boundary, 0) : end - boundary]

    def append_token(self, token_id: int) -> None:
        self.output_token_ids.append(int(token_id))

    # ------------------------------------------------------------------ progress
    def num_uncomputed_tokens(self) -> int:
        return len(self) - self.num_computed_tokens

    def is_prefilling(self) -> bool:
        return self.num_uncomputed_tokens() > 1

    def reset_for_recompute(self) -> None:
        """Preempted: the pages are gone, so every token is to run again; the tokens stay
        (clockwork/engine/sequence.py:79-82)."""
        self.num_computed_tokens = 0

    def is_finished(self) -> bool:
        return self.status in _FINISHED

    def __repr__(self) -> str:
        return (f"<Sequence {self.seq_id} {self.status.value}: {self.num_computed_tokens} of {len(self)} "
                f"tokens cached, {len(self.output_token_ids)} generated>")
