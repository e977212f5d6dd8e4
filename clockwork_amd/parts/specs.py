"""Specs of the built-in part kinds: their sizes and constants, nothing else.

Importing this module needs neither torch nor the HIP libraries, so
configuration code and CPU tests can build and inspect a model description.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Optional


@dataclass(frozen=True)
class RMSNormSpec:
    """y = weight * cast(x / sqrt(mean(x^2) + eps)); statistics in float32."""

    size: int
    eps: float


@dataclass(frozen=True)
class RopeNeoxSpec:
    """Rotary position encoding, half-split pairing (i, i + rotary_dim/2).

    inv_freq[j] = 1 / theta^(2j / rotary_dim); the first ``rotary_dim`` elements
    of each head are rotated, the rest pass through.
    """

    rotary_dim: int
    theta: float


@dataclass(frozen=True)
class AttentionSpec:
    """Softmax attention with grouped query heads over a paged key/value cache."""

    hidden_size: int
    num_heads: int
    num_kv_heads: int
    head_dim: int
    qkv_bias: bool
    out_bias: bool
    scale: float
    window: Optional[int] = None
    position: Any = None  # a position-encoding spec, or None for no encoding

    def __post_init__(self):
        if self.num_heads % self.num_kv_heads != 0:
            raise ValueError(
                f"num_heads {self.num_heads} is not a multiple of num_kv_heads {self.num_kv_heads}"
            )
        if self.head_dim % 16 != 0 or not 16 <= self.head_dim <= 256:
            raise ValueError(
                f"head_dim {self.head_dim} is not supported: the attention kernels take "
                "multiples of 16 from 16 to 256"
            )
        if self.window is not None and self.window < 1:
            raise ValueError(f"window must be positive, got {self.window}")


@dataclass(frozen=True)
class SwiGLUSpec:
    """down(silu(gate(x)) * up(x)), no biases."""

    hidden_size: int
    intermediate_size: int


@dataclass(frozen=True)
class TokenEmbeddingSpec:
    """The residual stream starts as row ``id`` of a [vocab, hidden] table: no scaling, nothing added."""

    vocab_size: int
    hidden_size: int


@dataclass(frozen=True)
class LinearHeadSpec:
    """logits = rows @ W^T with W [vocab, hidden], no bias, float32 logits. ``tied``: W is the
    embedding's table (one buffer, two uses) unless the checkpoint brings a head of its own."""

    vocab_size: int
    hidden_size: int
    tied: bool = False
