"""RMSNorm fused with the residual add (clockwork/engine/model.py:38-49, 147-152)."""

from __future__ import annotations

import torch

from clockwork_amd import ops
from clockwork_amd.config.spec import ParamSpec
from clockwork_amd.parts.base import Part
from clockwork_amd.parts.specs import RMSNormSpec


class RMSNorm(Part):
    graph_safe = True
    # takes a delta that is an ops.PendingPair (two branch outputs not yet added to the residual)
    accepts_pending = True
    def __init__(self, spec: RMSNormSpec) -> None:
        self.spec = spec

    def param_specs(self):
        return {"weight": ParamSpec((self.spec.size,), precision="stored", init=("one_plus_uniform", 0.1))}

    def bind(self, params, device, dtype) -> None:
        self.weight = params["weight"]
        self.dtype = dtype

    def forward(self, resid: torch.Tensor, delta, rows=None) -> torch.Tensor:
        n = resid.shape[0] if rows is None else rows.numel()
        out = torch.empty((n, self.spec.size), dtype=self.dtype, device=resid.device)
        return ops.add_rmsnorm(resid, delta, self.weight, self.spec.eps, out, rows)

    def lazy(self, resid: torch.Tensor, delta) -> "ops.LazyAddNorm":
        """The norm of resid + delta for a consumer that computes it inside its own kernel; the
        residual is not updated, so ``delta`` has to reach the next norm as well."""
        return ops.LazyAddNorm(resid, delta, self.weight, self.spec.eps, self.dtype)
