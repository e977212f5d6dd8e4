"""Grouped-query softmax attention over the paged cache (clockwork/engine/model.py:66-128).

Steps: one fused q/k/v product; bias, rotation and the cache write in one kernel (keys
and values of every token of the step are in the cache before any query reads it,
model.py:100); attention straight from the pages through the block table, prompt
portions and single tokens in the same step; output product.
"""

from __future__ import annotations

import torch

from clockwork_amd import ops
from clockwork_amd.config.spec import KVPagesSpec, ParamSpec
from clockwork_amd.parts.base import EntryCache, Part
from clockwork_amd.parts.rope import NoPosition
from clockwork_amd.parts.specs import AttentionSpec
from clockwork_amd.registry import build_part


class PagedAttention(Part):
    @property
    def graph_safe(self) -> bool:
        """A fixed sequence of launches if the position encoding is one too."""
        return bool(getattr(self.position, "graph_safe", False))

    def __init__(self, spec: AttentionSpec) -> None:
        self.spec = spec
        self.position = build_part(spec.position) if spec.position is not None else NoPosition()
        self.q_width = spec.num_heads * spec.head_dim
        self.kv_width = spec.num_kv_heads * spec.head_dim

    def param_specs(self):
        s = self.spec
        width = self.q_width + 2 * self.kv_width
        specs = {
            "qkv_weight": ParamSpec((width, s.hidden_size)),
            "out_weight": ParamSpec((s.hidden_size, self.q_width)),
        }
        if s.qkv_bias:
            specs["qkv_bias"] = ParamSpec((width,), precision="stored", init=("normal", 0.02))
        if s.out_bias:
            specs["out_bias"] = ParamSpec((s.hidden_size,), precision="compute", init=("normal", 0.02))
        return specs

    def cache_need(self):
        return KVPagesSpec(self.spec.num_kv_heads, self.spec.head_dim, self.spec.window)

    def bind(self, params, device, dtype) -> None:
        self.qkv_weight = params["qkv_weight"]
        self.qkv_bias = params.get("qkv_bias")
        self.out_weight = params["out_weight"]
        self.out_bias = params.get("out_bias")
        self.position.bind({}, device, dtype)

    def forward(self, x: torch.Tensor, ctx, cache: EntryCache) -> torch.Tensor:
        s = self.spec
        nh, nkv, hd = s.num_heads, s.num_kv_heads, s.head_dim
        T = x.shape[0]
        fused = getattr(self.position, "project_rotate_store", None) if cache.writes else None
        qkv = None
        if fused is not None:
            qkv = fused(x, self.qkv_weight, self.qkv_bias, ctx.positions, ctx.slots[cache.group], nh, nkv, hd, cache.k, cache.v)
        if qkv is not None:
            pass  # q only, [T, nh * hd]: keys and values are in the cache already
        elif cache.writes:
            qkv = ops.linear(x, self.qkv_weight)
            self.position.rotate_and_store(
                qkv, self.qkv_bias, ctx.positions, ctx.slots[cache.group], nh, nkv, hd, cache.k, cache.v
            )
        else:
            # the keys and values of another entry are read: only queries are made here
            qkv = ops.linear(x, self.qkv_weight[: self.q_width])
            bias = self.qkv_bias[: self.q_width] if self.qkv_bias is not None else None
            self.position.rotate_and_store(qkv, bias, ctx.positions, None, nh, 0, hd, None, None)
        out = torch.empty((T, self.q_width), dtype=x.dtype, device=x.device)
        mfma = ops.prefill_attention_supported(hd, x.dtype)
        plan = ctx.attention_plan(nh, nkv, narrow_ok=mfma and ops.prefill_row_blocks_ok(hd, 2))
        common = dict(
            q=qkv, q_stride=qkv.shape[1], out=out, k_cache=cache.k, v_cache=cache.v,
            block_tables=ctx.block_tables[cache.group], ctx_lens=ctx.ctx_lens, cu_q=ctx.cu_q,
            nh=nh, nkv=nkv, hd=hd, block_size=cache.block_size, window=s.window or 0,
            scale=s.scale, n_tokens=T, n_requests=ctx.num_requests,
        )
        if plan.n_wide and mfma:
            ops.attention_prefill(items=plan.mfma_items, n_items=plan.n_mfma, row_blocks=plan.mfma_row_blocks, **common)
        elif plan.n_wide:
            ops.attention(items=plan.wide_items, n_items=plan.n_wide, rows=64, gh=plan.gh_wide,
                          n_splits=1, **common)
        if plan.n_single and ops.decode_attention_supported(hd, x.dtype):
            workspace = None
            if plan.decode_splits > 1:
                need = ops.decode_attention_workspace_floats(hd, plan.n_single, nh, nkv, plan.decode_splits)
                workspace = torch.empty(need, dtype=torch.float32, device=x.device)
            ops.attention_decode(items=plan.single_items, n_items=plan.n_single, n_splits=plan.decode_splits,
                                 workspace=workspace, identity=plan.single_identity,
                                 split_keys=plan.decode_split_keys, max_ctx=plan.decode_max_ctx, **common)
        elif plan.n_single:
            workspace = None
            if plan.single_splits > 1:
                need = ops.attention_workspace_floats(hd, 16, plan.n_single, nkv, plan.chunks_single, plan.single_splits)
                workspace = torch.empty(need, dtype=torch.float32, device=x.device)
            ops.attention(items=plan.single_items, n_items=plan.n_single, rows=16, gh=plan.gh_single,
                          n_splits=plan.single_splits, workspace=workspace, **common)
        return ops.linear(out, self.out_weight, self.out_bias, partial_ok=True)
