"""Interfaces of the parts a model is put together from.

A part is built from its spec alone (sizes and constants are parameters; no part
knows which model it is in) and goes through three stages:

1. ``param_specs()`` - the tensors it owns: ``{local name: ParamSpec}``. Needs no GPU.
2. ``bind(params, device, dtype)`` - receives ``{local name: device tensor}`` and
   prepares whatever else it needs on the device (tables, constants).
3. its run method, called during a step.

Roles and their run methods:

* embedding:     ``forward(ctx) -> resid``: the float32 residual stream [T, H] of the step's
                 tokens (``ctx.token_ids``, ``ctx.positions``). May offer ``table()``, the
                 [vocab, H] matrix a tied head uses, and ``positions(ctx) -> tensor``: what
                 ``ctx.positions`` holds for the parts of this step (an offset, several axes a
                 token), made on the device from ``ctx.sequence_positions`` (int32 [T], each
                 token's index in its request) before anything else runs; without it
                 ``ctx.positions`` is ``ctx.sequence_positions``.
* norm:          ``forward(resid, delta, rows=None) -> normed`` - ``resid`` is the
                 float32 residual stream [T, H]; ``delta`` (activation type, an
                 ``ops.PartialSums`` of that shape, or None)
                 is added to it in place first; returns the normed rows in the
                 activation type. With ``rows`` only those rows are produced and
                 ``resid`` is left untouched.
* mixer:         ``forward(x, ctx, cache) -> y`` with x, y [T, H] in the activation
                 type (y may be an ``ops.PartialSums``: it only ever goes to a norm); ``cache_need()`` returns a KVPagesSpec, a StateSpec or None.
                 ``cache`` is the run entry's :class:`EntryCache`.
* feed-forward:  ``forward(x, ctx) -> y``.
* position enc.: used by a mixer, not by the block; the attention mixer expects
                 ``rotate_and_store(qkv, bias, positions, slots, nh, nkv, hd, k, v)``, and
                 uses ``project_rotate_store(x, weight, bias, positions, slots, nh, nkv, hd,
                 k, v) -> q or None`` when the part offers it (product, encoding and cache
                 write in one kernel).
* arrangement:   built by its factory from the block's parts as keyword arguments, under
                 the names the ``LayerSpec`` gives them (``mixer``, ``feed_forward``,
                 ``mixer_norm``, ``ffn_norm`` or any others). ``parts() -> {name: part}``;
                 ``forward(resid, delta, ctx, cache) -> delta`` wires norms, mixer and
                 feed-forward around the residual stream; the returned ``delta`` is the last
                 branch output, not yet added. The part named ``mixer`` owns the block's
                 cache. Optional ``first_norm() -> part``: the norm that takes the delta handed
                 on; if it has ``accepts_pending`` the block before may hand on two outputs
                 (``ops.PendingPair``), without the hook it hands on one.
* head:          ``forward(rows, ctx) -> logits``: float32 [n, vocab] for the final norm's rows.
                 A head whose spec has ``tied`` set gets ``use_embedding(embedding part)``
                 before ``bind``. ``matrices()``: what a step streams through it (byte counts).

What any part may add:

* ``graph_safe = True``: its step is a fixed sequence of launches on the device (no host
  reads, no shapes that depend on data), so a step may be captured as a HIP graph.
* ``prepare(ctx)``: make, before ``forward``, what depends on the step's shape alone (work
  items, uploaded through ``ctx.upload``) and keep it in ``ctx.plans``; a captured step is
  prepared once, outside the capture.
* ``shape_class(q_lens, ctx_lens)``: a label for what of a step's shape decides which kernels
  the part launches; a captured graph serves steps of its own class.
* ``kernel_libraries()``: the HIP libraries it runs, as (name, head size or None).

Fixed-size state: ``cache.state`` is [slots, *shape] of the run entry; a request's row is
``ctx.state_slots[r]`` (``ctx.h_state_slots`` on the host). Rows of a fixed-shape batch that
hold no request carry the pool's spare last slot, so a part may read and write every row's
slot; the state of a request whose first token runs in the step is cleared before the parts run.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Optional

from clockwork_amd.config.spec import ParamSpec


class Part:
    """Convenience base: no parameters, nothing to prepare."""

    def param_specs(self) -> dict[str, ParamSpec]:
        return {}

    def bind(self, params: dict, device, dtype) -> None:
        self.params = params

    def cache_need(self) -> Optional[Any]:
        return None


@dataclass
class EntryCache:
    """The cache of one run entry as its mixer sees it.

    Key/value kind: ``k`` and ``v`` are flat [num_blocks * block_size, kv_heads, head_dim]
    views of the entry's pages, ``group`` indexes the step context's per-group block
    tables and slot mappings, ``writes`` is False when the entry reads another entry's
    cache. A mixer with planes of its own (``PagedRowsSpec``) finds each in ``planes`` by name,
    a flat [num_blocks * block_size, *row shape] view addressed the same way. State kind:
    ``state`` is [slots, *shape]; the request's row is ``ctx.state_slots[r]``.
    """

    group: int = -1
    k: Any = None
    v: Any = None
    planes: Any = None   # {plane name: flat view}: ``k`` and ``v`` among them, or a mixer's own
    state: Any = None
    writes: bool = True
    block_size: int = 0
