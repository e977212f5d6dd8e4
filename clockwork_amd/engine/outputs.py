"""What the engine hands back for a request after a step."""

from __future__ import annotations

from dataclasses import dataclass
from typing import Optional


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
