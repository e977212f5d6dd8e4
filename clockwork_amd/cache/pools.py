"""Device memory behind the cache manager's bookkeeping.

Per key/value group one tensor [entries, 2 (keys, values), num_blocks, block_size,
kv_heads, head_dim] in the engine's dtype: an entry's keys (or values) are the
reference's paged layout [num_blocks, block_size, kv_heads, head_dim]
(clockwork/kvcache/kv_cache.py:24-30), one page id addresses the same page in
every entry of the group, and a copy-on-write copies all of them with one kernel.
A paged group with planes of a mixer's own (``PagedRowsSpec``) is laid out the same way when
its planes' rows are of one shape, [entries, planes, num_blocks, block_size, *row]; planes of
different shapes get a tensor each, [entries, num_blocks, block_size, *row].
Per state group one tensor [entries, max_num_seqs + 2, *shape]: a slot per live request, a
spare one that belongs to nobody (rows of a fixed-shape batch that hold no request point there,
so a part may read and write "its" slot for every row without asking) and, last, the template
of a fresh state, which a request's slot is set to when its first token arrives.
"""

from __future__ import annotations

import torch

from clockwork_amd import ops
from clockwork_amd.cache.manager import GroupLayout
from clockwork_amd.parts.base import EntryCache


def _row_elements(shape) -> int:
    n = 1
    for d in shape:
        n *= int(d)
    return n


def page_bytes(groups: list[GroupLayout], block_size: int, dtype: torch.dtype) -> int:
    """Bytes one page number occupies: every plane's rows (keys and values, or a mixer's own) in
    every entry of every paged group (each group has a pool of ``num_blocks`` pages of its own)."""
    elem = torch.empty((), dtype=dtype).element_size()
    total = 0
    for group in groups:
        if group.is_kv:
            per_token = sum(_row_elements(shape) for _, shape in group.need.planes)
            total += len(group.entries) * block_size * per_token * elem
    return total


def pages_that_fit(groups: list[GroupLayout], block_size: int, dtype: torch.dtype, free_bytes: int,
                   fraction: float, most: int) -> int:
    """How many pages per group to make when the configuration leaves it open: ``fraction`` of
    the free device memory, but no more than ``most`` (what the scheduler can ever hold live,
    with room for cached prefixes) and at least one page."""
    per_page = page_bytes(groups, block_size, dtype)
    if per_page == 0:
        return 1
    if not 0.0 < fraction <= 1.0:
        raise ValueError(f"memory_fraction must be in (0, 1], got {fraction}")
    fit = int(free_bytes * fraction) // per_page
    if fit < 1:
        raise RuntimeError(
            f"no room for the cache: one page takes {per_page} bytes, {free_bytes} bytes of device memory are free"
        )
    return max(1, min(fit, most))


class CachePools:
    def __init__(self, groups: list[GroupLayout], block_size: int, num_blocks: int,
                 max_num_seqs: int, dtype: torch.dtype, device, fill: float = 0.0) -> None:
        self.groups = groups
        self.block_size = block_size
        self.num_blocks = num_blocks
        self.max_num_seqs = max_num_seqs
        # per paged group: one tensor [entries, planes, num_blocks, block_size, *row] when every
        # plane's row has the same shape (keys and values do), else None
        self.kv: list = []
        # per paged group: {plane name: [entries, num_blocks, block_size, *row]} (views of the
        # tensor above, or tensors of their own)
        self.planes: list[dict] = []
        self.state: list[torch.Tensor] = []
        self._kv_index: dict[int, tuple[int, int]] = {}     # run entry -> (paged group, row)
        self._state_index: dict[int, tuple[int, int]] = {}  # run entry -> (state group, row)
        for group in groups:
            need = group.need
            if group.is_kv:
                names = [name for name, _ in need.planes]
                shapes = [tuple(int(d) for d in shape) for _, shape in need.planes]
                if all(shape == shapes[0] for shape in shapes):
                    pool = torch.full((len(group.entries), len(names), num_blocks, block_size, *shapes[0]), fill,
                                      dtype=dtype, device=device)
                    planes = {name: pool[:, i] for i, name in enumerate(names)}
                else:
                    pool = None
                    planes = {name: torch.full((len(group.entries), num_blocks, block_size, *shape), fill, dtype=dtype,
                                               device=device) for name, shape in zip(names, shapes)}
                for row, entry in enumerate(group.entries):
                    self._kv_index[entry] = (len(self.kv), row)
                self.kv.append(pool)
                self.planes.append(planes)
            else:
                shape = (len(group.entries), max_num_seqs + 2, *need.shape)
                pool = torch.zeros(shape, dtype=getattr(torch, need.dtype), device=device)
                if need.init[0] == "fill":
                    pool.fill_(need.init[1])
                if (pool[0, 0].numel() * pool.element_size()) % 4:
                    raise ValueError(f"a state of shape {tuple(need.shape)} {need.dtype} is not a whole number of "
                                     "32-bit words: the kernel that sets a fresh request's state takes words")
                for row, entry in enumerate(group.entries):
                    self._state_index[entry] = (len(self.state), row)
                self.state.append(pool)

    def bytes(self) -> int:
        paged = [t for planes in self.planes for t in planes.values()]
        return sum(t.numel() * t.element_size() for t in paged + self.state)

    def kv_bytes_per_token(self) -> int:
        """Bytes one cached token occupies in the pages, all groups, entries and planes."""
        total = 0
        for planes in self.planes:
            for t in planes.values():
                total += t.shape[0] * t[0, 0, 0].numel() * t.element_size()
        return total

    def entry_cache(self, entry: int, source: int | None = None) -> EntryCache:
        """The cache of run entry ``entry``; with ``source`` the entry reads that entry's cache."""
        owner = entry if source is None else source
        if owner in self._kv_index:
            g, row = self._kv_index[owner]
            flat = {name: t[row].reshape(-1, *t.shape[3:]) for name, t in self.planes[g].items()}
            return EntryCache(group=g, k=flat.get("k"), v=flat.get("v"), planes=flat, writes=source is None,
                              block_size=self.block_size)
        if owner in self._state_index:
            g, row = self._state_index[owner]
            return EntryCache(group=g, state=self.state[g][row], writes=source is None)
        return EntryCache(writes=False)

    def set_fresh_state(self, entry: int, value: torch.Tensor) -> None:
        """Make ``value`` what run entry ``entry``'s state begins as for every new request (a
        part with a beginning of its own calls this once its parameters are bound)."""
        g, row = self._state_index[entry]
        self.state[g][row, self.max_num_seqs + 1].copy_(value)

    def copy_pages(self, group: int, pairs: list[tuple[int, int]]) -> None:
        """Copy page src -> dst in every entry and plane of the group."""
        if not pairs:
            return
        pool = self.kv[group]
        tensors = [pool.view(pool.shape[0] * pool.shape[1], pool.shape[2], -1)] if pool is not None else [
            t.view(t.shape[0], t.shape[1], -1) for t in self.planes[group].values()]
        index = torch.tensor(pairs, dtype=torch.int32, device=tensors[0].device)
        for planes in tensors:
            ops.copy_pages(planes, index)

    def copy_state(self, src_slot: int, dst_slot: int) -> None:
        for pool in self.state:
            pool[:, dst_slot].copy_(pool[:, src_slot])

    def set_fresh_states(self, state_slots: torch.Tensor, starts: torch.Tensor, n: int) -> None:
        """Set the state of the step's requests that begin at position 0 to the fresh state: the
        pool's template row, zeros unless the spec or a part says otherwise (device int32 arrays of
        the step: each request's slot and first position). One kernel per state group; part of
        every step of a model with state, captured or not."""
        for pool in self.state:
            ops.fresh_state_rows(pool, state_slots, starts, n)
