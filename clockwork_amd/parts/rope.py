"""Rotary position encoding, half-split pairs, fused with the key/value cache write.

inv_freq follows the reference's formula exactly, evaluated on the host in float32
(clockwork/engine/model.py:171-175), so angles pos * inv_freq match it bit for bit;
the rotation itself (model.py:32-35, 92-95) runs in float32 inside the kernel.
"""

from __future__ import annotations

import torch

from clockwork_amd import ops
from clockwork_amd.parts.base import Part
from clockwork_amd.parts.specs import RopeNeoxSpec


class RopeNeox(Part):
    graph_safe = True

    def __init__(self, spec: RopeNeoxSpec) -> None:
        if spec.rotary_dim % 2:
            raise ValueError(f"rotary_dim {spec.rotary_dim} must be even")
        self.spec = spec

    def bind(self, params, device, dtype) -> None:
        d = self.spec.rotary_dim
        inv_freq = 1.0 / (self.spec.theta ** (torch.arange(0, d, 2, dtype=torch.float32) / d))
        self.inv_freq = inv_freq.to(device)

    def rotate_and_store(self, qkv, bias, positions, slots, nh, nkv, hd, k_cache, v_cache) -> None:
        if self.spec.rotary_dim > hd:
            raise ValueError(f"rotary_dim {self.spec.rotary_dim} exceeds head_dim {hd}")
        ops.rope_kv_write(qkv, bias, positions, slots, self.inv_freq, self.spec.rotary_dim, nh, nkv, hd, k_cache, v_cache)


    def project_rotate_store(self, x, weight, bias, positions, slots, nh, nkv, hd, k_cache, v_cache):
        """Optional fast path of the attention mixer: the q/k/v product, this encoding and the cache
        write as one kernel. Returns q [T, nh * hd], or None when the shapes do not allow it (the
        mixer then runs the product and ``rotate_and_store`` apart)."""
        if slots is None or not ops.qkv_rope_fused_supported(x, weight, self.spec.rotary_dim, hd):
            return None
        return ops.qkv_rope_fused(x, weight, bias, positions, slots, self.inv_freq, nh, nkv, hd, k_cache, v_cache)


class NoPosition(Part):
    """Stands in when a mixer has no position encoding: bias and cache write only."""

    graph_safe = True

    def rotate_and_store(self, qkv, bias, positions, slots, nh, nkv, hd, k_cache, v_cache) -> None:
        ops.rope_kv_write(qkv, bias, positions, slots, None, 0, nh, nkv, hd, k_cache, v_cache)
