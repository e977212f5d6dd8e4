"""Dense SwiGLU feed-forward: down(silu(gate(x)) * up(x)) (clockwork/engine/model.py:52-63).

gate and up are one product over a fused [2 I, H] weight; the gate multiply is one kernel.
"""

from __future__ import annotations

import torch

from clockwork_amd import ops
from clockwork_amd.config.spec import ParamSpec
from clockwork_amd.parts.base import Part
from clockwork_amd.parts.specs import SwiGLUSpec


class SwiGLU(Part):
    graph_safe = True
    def __init__(self, spec: SwiGLUSpec) -> None:
        self.spec = spec

    def param_specs(self):
        H, I = self.spec.hidden_size, self.spec.intermediate_size
        return {"gate_up_weight": ParamSpec((2 * I, H)), "down_weight": ParamSpec((H, I))}

    def bind(self, params, device, dtype) -> None:
        self.gate_up = params["gate_up_weight"]
        self.down = params["down_weight"]

    def fuses_input_norm(self, n_tokens: int, dtype, delta) -> bool:
        """True if ``forward`` can take an ``ops.LazyAddNorm`` of that many rows and make the
        norm inside the gate/up product (decode: few rows)."""
        H, I = self.spec.hidden_size, self.spec.intermediate_size
        return ops.swiglu_norm_fusable(n_tokens, 2 * I, H, dtype, self.gate_up, delta)

    def forward(self, x, ctx) -> torch.Tensor:
        policy = getattr(ctx, "products", None)
        return ops.linear(ops.linear_swiglu(x, self.gate_up, policy=policy), self.down, partial_ok=True, policy=policy)
