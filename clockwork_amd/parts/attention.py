"""Grouped-query softmax attention over the paged cache (clockwork/engine/model.py:66-128).

Steps: one fused q/k/v product; bias, rotation and the cache write in one kernel (keys
and values of every token of the step are in the cache before any query reads it,
model.py:100); attention straight from the pages through the block table, prompt
portions and single tokens in the same step; output product.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import numpy as np
import torch

from clockwork_amd import ops
from clockwork_amd.config.spec import KVPagesSpec, ParamSpec
from clockwork_amd.parts.base import EntryCache, Part
from clockwork_amd.parts.rope import NoPosition
from clockwork_amd.parts.specs import AttentionSpec
from clockwork_amd.registry import build_part


@dataclass
class AttentionPlan:
    """Work items of the attention kernels for one head geometry (see csrc/attention.hip).

    Requests with one token go to the 16-row kernel, cut over their keys into
    ``single_splits`` parts; longer portions are cut into tiles of the 64-row kernel."""

    wide_items: Optional[torch.Tensor] = None
    n_wide: int = 0
    gh_wide: int = 1
    wide_splits: int = 1       # parts every wide item's key range is cut into (few items with many keys)
    mfma_items: Optional[torch.Tensor] = None   # the same portions cut for the bfloat16 matrix-core kernel
    n_mfma: int = 0
    mfma_row_blocks: int = 4   # row blocks of that kernel's workgroups: 2 when 4 would leave compute units idle
    mfma_parts: int = 1        # the most parts an item's key range is shared among (1: no item is cut)
    single_items: Optional[torch.Tensor] = None
    n_single: int = 0
    gh_single: int = 1
    chunks_single: int = 1
    single_splits: int = 1
    decode_splits: int = 1   # splits of the bfloat16 decode kernel (finer: it walks 16-key tiles)
    decode_split_keys: int = 0    # keys of each of those splits, at fixed places (a multiple of 32)
    decode_max_ctx: int = 0       # the longest context the fixed places were planned for
    single_identity: bool = False  # a batch of single tokens only: item i is request i, token row i


# a portion's key ranges count as long when its tokens see this many keys or more on average
LONG_RANGE_KEYS = 3072


def portions_have_short_ranges(q_lens, ctx_lens) -> bool:
    """The rule by which a step's portions (entries of more than one token) choose the shape of
    the matrix-core kernel's workgroups: True while their tokens see fewer than 3072 keys on
    average. Behind a long cached prefix every workgroup's key range is long and about the same,
    and sharing the keys among more rows wins (2048 tokens of the 1.5B shape: 46 against 52 us
    with no prefix, 94 against 96 us behind 2048 tokens, 197 against 182 us behind 6144)."""
    tokens = sum(q for q in q_lens if q > 1)
    keys = sum(q * (c - q / 2.0) for q, c in zip(q_lens, ctx_lens) if q > 1)
    return tokens > 0 and keys / tokens < LONG_RANGE_KEYS


# a part of an item's key range is at least this many keys (two stages of the kernel), and an item
# is cut into at most this many parts
MIN_PART_KEYS = 256
MAX_PARTS = 64


def _share_long_key_ranges(items: np.ndarray, ctx, workgroups_per_item: int):
    """A compute unit holds one workgroup of the kernel for portions at a time (its tiles fill the
    unit's LDS), so a launch with fewer workgroups than half the compute units (a short portion behind a long cached
    prefix: the end of a long prompt, a new turn of a long conversation) leaves most of the card
    idle while a few units walk through thousands of keys. Such a launch's items stand in the
    list once for each of several parts, one after the other, as ``part | parts << 8`` in the
    fourth field; the kernel gives each part a run of the item's keys and a second kernel puts
    them together. Launches that fill the card are left alone: there the parts cost more than
    they bring (measured). Returns the flat item list and the most parts of an item (1: nothing
    was cut)."""
    workgroups = len(items) * workgroups_per_item
    spare = ctx.num_compute_units // max(workgroups, 1)
    if len(items) == 0 or spare < 2:
        return items.reshape(-1), 1
    ctx_lens = np.asarray(ctx.h_ctx_lens, dtype=np.int64)
    q_lens = np.asarray(ctx.h_q_lens, dtype=np.int64)
    req = items[:, 0]
    keys = ctx_lens[req] - q_lens[req] + items[:, 1] + items[:, 2]  # keys that the item's last token sees
    parts = np.minimum(spare, keys // MIN_PART_KEYS).clip(1, MAX_PARTS).astype(np.int64)
    most = int(parts.max())
    if most == 1:
        return items.reshape(-1), 1
    out = np.repeat(items, parts, axis=0)
    first = np.cumsum(parts) - parts  # where each item's parts begin
    part = np.arange(len(out)) - np.repeat(first, parts)
    out[:, 3] = part | (np.repeat(parts, parts) << 8)
    return out.astype(np.int32).reshape(-1), most


def attention_plan(ctx, nh: int, nkv: int, narrow_ok: bool = False) -> AttentionPlan:
    """The step's work items for heads of this geometry, made once a step and kept in
    ``ctx.plans``. ``narrow_ok``: the matrix-core kernel for portions also comes with two row
    blocks a workgroup (see ``ops.prefill_row_blocks_ok``)."""
    # a batch of single tokens has no portions: one plan, whatever the kernel for portions offers
    narrow_ok = bool(narrow_ok) and any(q > 1 for q in ctx.h_q_lens)
    key = ("attention", nh, nkv, narrow_ok)
    plan = ctx.plans.get(key)
    if plan is None:
        plan = ctx.plans[key] = _make_plan(ctx, nh, nkv, narrow_ok)
    return plan


def _make_plan(ctx, nh: int, nkv: int, narrow_ok: bool) -> AttentionPlan:
    group = nh // nkv
    gh_wide = min(group, 64)
    tokens_per_tile = 64 // gh_wide
    gh_single = min(group, 16)
    wide: list = []   # one array of items per portion
    mfma: list = []
    # Workgroups of four row blocks share each key among the most rows, but a launch has to
    # fill the compute units, and the workgroup with the longest key range decides its time:
    # with fewer than 1.5 workgroups a compute unit, halve them (unless the key ranges are long).
    tokens_of_four = 4 * (32 // min(group, 32))
    workgroups = sum(-(-q // tokens_of_four) for q in ctx.h_q_lens if q > 1) * nkv * -(-group // 32)
    short_ranges = portions_have_short_ranges(ctx.h_q_lens, ctx.h_ctx_lens)
    row_blocks = 2 if narrow_ok and short_ranges and 2 * workgroups < 3 * ctx.num_compute_units else 4
    tokens_per_mfma_item = row_blocks * (32 // min(group, 32))
    single: list[int] = []
    longest_single = 0

    def items_of(r: int, q_len: int, step: int, longest_first: bool) -> np.ndarray:
        """(request, first token, tokens, 0) for runs of ``step`` tokens of one portion."""
        tok0 = np.arange(0, q_len, step, dtype=np.int32)
        if longest_first:
            tok0 = tok0[::-1]
        out = np.zeros((tok0.size, 4), dtype=np.int32)
        out[:, 0] = r
        out[:, 1] = tok0
        out[:, 2] = np.minimum(step, q_len - tok0)
        return out.reshape(-1)

    for r, q_len in enumerate(ctx.h_q_lens):
        if q_len == 1:
            single += [r, 0, 1, 0]
            longest_single = max(longest_single, ctx.h_ctx_lens[r])
        else:
            wide.append(items_of(r, q_len, tokens_per_tile, False))
            # longest key ranges first: the last tokens of a portion have the most work
            mfma.append(items_of(r, q_len, tokens_per_mfma_item, True))
    wide = np.concatenate(wide) if wide else np.zeros(0, dtype=np.int32)
    mfma = np.concatenate(mfma) if mfma else np.zeros(0, dtype=np.int32)
    plan = AttentionPlan(gh_wide=gh_wide, gh_single=gh_single, mfma_row_blocks=row_blocks)
    mfma, plan.mfma_parts = _share_long_key_ranges(mfma.reshape(-1, 4), ctx, nkv * -(-group // 32))
    plan.n_wide, plan.n_single, plan.n_mfma = len(wide) // 4, len(single) // 4, len(mfma) // 4
    if plan.n_wide:
        # the 64-row kernel cuts every item's keys the same number of ways: as many as there are idle
        # compute units for, while the longest portion's keys give each part MIN_PART_KEYS
        spare = ctx.num_compute_units // (plan.n_wide * nkv * -(-group // gh_wide))
        most_keys = max(c for q, c in zip(ctx.h_q_lens, ctx.h_ctx_lens) if q > 1)
        plan.wide_splits = int(max(1, min(spare, most_keys // MIN_PART_KEYS, MAX_PARTS)))
    plan.chunks_single = -(-group // gh_single)
    if plan.n_single:
        groups_running = plan.n_single * nkv * plan.chunks_single
        by_occupancy = -(-4 * ctx.num_compute_units // groups_running)
        by_length = max(1, longest_single // 256)
        plan.single_splits = max(1, min(by_occupancy, by_length, 64))
        # decode kernel: a workgroup per (request, kv head, split); a split is at least 128 keys
        # (one 32-key tile for each of its four waves). As many splits as still give every
        # workgroup a compute unit of its own: one more and some units run a second round (24
        # requests of 2100 keys on 2 kv heads, kernel and merge: 19.2 us with 4 splits, 22.4 with 6;
        # 96 requests: 42.5 us with 1, 50.6 with 3). More than 64 splits never paid: one request
        # with 30000 keys takes 16 us with 64 to 128 splits and 19 us with 235.
        base = plan.n_single * nkv * -(-group // min(group, 16))
        plan.decode_splits = max(1, min(ctx.num_compute_units // base, longest_single // 128, 64))
        # fixed places for the splits: a workgroup then knows its pages before it knows the
        # request's length, which saves it a trip to memory
        plan.decode_split_keys = 32 * -(-(-(-longest_single // plan.decode_splits)) // 32)
        plan.decode_max_ctx = longest_single
        plan.single_identity = plan.n_single == len(ctx.h_q_lens)
    plan.wide_items, plan.single_items, plan.mfma_items = ctx.upload([wide, single, mfma])
    return plan


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

    def kernel_libraries(self) -> list:
        return [("attention", int(self.spec.head_dim))]

    def _plan(self, ctx, dtype) -> AttentionPlan:
        hd = self.spec.head_dim
        narrow_ok = ops.prefill_attention_supported(hd, dtype) and ops.prefill_row_blocks_ok(hd, 2)
        return attention_plan(ctx, self.spec.num_heads, self.spec.num_kv_heads, narrow_ok=narrow_ok)

    def prepare(self, ctx) -> None:
        """The step's work items, before ``forward`` (a captured step must not make them)."""
        self._plan(ctx, self.dtype)

    def shape_class(self, q_lens, ctx_lens):
        """Portions behind a long cached prefix run another workgroup shape than early ones."""
        if not any(q > 1 for q in q_lens):
            return "single tokens"
        return "short key ranges" if portions_have_short_ranges(q_lens, ctx_lens) else "long key ranges"

    def bind(self, params, device, dtype) -> None:
        self.qkv_weight = params["qkv_weight"]
        self.qkv_bias = params.get("qkv_bias")
        self.out_weight = params["out_weight"]
        self.out_bias = params.get("out_bias")
        self.dtype = dtype
        self.position.bind({}, device, dtype)

    def forward(self, x: torch.Tensor, ctx, cache: EntryCache) -> torch.Tensor:
        s = self.spec
        nh, nkv, hd = s.num_heads, s.num_kv_heads, s.head_dim
        policy = getattr(ctx, "products", None)
        fused = getattr(self.position, "project_rotate_store", None) if cache.writes else None
        qkv = None
        if fused is not None:
            qkv = fused(x, self.qkv_weight, self.qkv_bias, ctx.positions, ctx.slots[cache.group], nh, nkv, hd, cache.k, cache.v)
        if qkv is not None:
            pass  # q only, [T, nh * hd]: keys and values are in the cache already
        elif cache.writes:
            qkv = ops.linear(x, self.qkv_weight, policy=policy)
            self.position.rotate_and_store(
                qkv, self.qkv_bias, ctx.positions, ctx.slots[cache.group], nh, nkv, hd, cache.k, cache.v
            )
        else:
            # the keys and values of another entry are read: only queries are made here
            qkv = ops.linear(x, self.qkv_weight[: self.q_width], policy=policy)
            bias = self.qkv_bias[: self.q_width] if self.qkv_bias is not None else None
            self.position.rotate_and_store(qkv, bias, ctx.positions, None, nh, 0, hd, None, None)
        out = self.attend(qkv, ctx, cache)
        return ops.linear(out, self.out_weight, self.out_bias, partial_ok=True, policy=policy)

    def attend(self, q: torch.Tensor, ctx, cache: EntryCache) -> torch.Tensor:
        """Attention of the step's rotated queries (the first ``num_heads * head_dim`` columns of
        ``q``, one row a token) over the keys and values that ``cache`` holds, [T, heads * head_dim]:
        the kernels and work items that the step's plan names, and nothing else of the layer."""
        s = self.spec
        nh, nkv, hd = s.num_heads, s.num_kv_heads, s.head_dim
        T = q.shape[0]
        out = torch.empty((T, self.q_width), dtype=q.dtype, device=q.device)
        mfma = ops.prefill_attention_supported(hd, q.dtype)
        plan = self._plan(ctx, q.dtype)
        common = dict(
            q=q, q_stride=q.shape[1], out=out, k_cache=cache.k, v_cache=cache.v,
            block_tables=ctx.block_tables[cache.group], ctx_lens=ctx.ctx_lens, cu_q=ctx.cu_q,
            nh=nh, nkv=nkv, hd=hd, block_size=cache.block_size, window=s.window or 0,
            scale=s.scale, n_tokens=T, n_requests=ctx.num_requests,
        )
        if plan.n_wide and mfma:
            workspace = None
            if plan.mfma_parts > 1:
                need = ops.prefill_attention_workspace_floats(hd, plan.n_mfma, nh, nkv, plan.mfma_row_blocks)
                workspace = torch.empty(need, dtype=torch.float32, device=q.device)
            ops.attention_prefill(items=plan.mfma_items, n_items=plan.n_mfma, row_blocks=plan.mfma_row_blocks,
                                  workspace=workspace, **common)
        elif plan.n_wide:
            workspace = None
            if plan.wide_splits > 1:
                need = ops.attention_workspace_floats(hd, 64, plan.n_wide, nkv, -(-(nh // nkv) // plan.gh_wide), plan.wide_splits)
                workspace = torch.empty(need, dtype=torch.float32, device=q.device)
            ops.attention(items=plan.wide_items, n_items=plan.n_wide, rows=64, gh=plan.gh_wide,
                          n_splits=plan.wide_splits, workspace=workspace, **common)
        if plan.n_single and ops.decode_attention_supported(hd, q.dtype):
            workspace = None
            if plan.decode_splits > 1:
                need = ops.decode_attention_workspace_floats(hd, plan.n_single, nh, nkv, plan.decode_splits)
                workspace = torch.empty(need, dtype=torch.float32, device=q.device)
            ops.attention_decode(items=plan.single_items, n_items=plan.n_single, n_splits=plan.decode_splits,
                                 workspace=workspace, identity=plan.single_identity,
                                 split_keys=plan.decode_split_keys, max_ctx=plan.decode_max_ctx, **common)
        elif plan.n_single:
            workspace = None
            if plan.single_splits > 1:
                need = ops.attention_workspace_floats(hd, 16, plan.n_single, nkv, plan.chunks_single, plan.single_splits)
                workspace = torch.empty(need, dtype=torch.float32, device=q.device)
            ops.attention(items=plan.single_items, n_items=plan.n_single, rows=16, gh=plan.gh_single,
                          n_splits=plan.single_splits, workspace=workspace, **common)
        return out
