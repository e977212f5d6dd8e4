"""Device memory behind the cache manager's bookkeeping.

Per key/value group one tensor [entries, 2 (keys, values), num_blocks, block_size,
kv_heads, head_dim] in the engine's dtype: an entry's keys (or values) are the
reference's paged layout [num_blocks, block_size, kv_heads, head_dim]
(clockwork/kvcache/kv_cache.py:24-30), one page id addresses the same page in
every entry of the group, and a copy-on-write copies all of them with one kernel.
Per state group one tensor [entries, max_num_seqs + 1, *shape]: a slot per live request and a
spare one at the end that belongs to nobody (rows of a fixed-shape batch that hold no request
point there, so a part may read and write "its" slot for every row without asking).
"""

from __future__ import annotations

import torch

from clockwork_amd import ops
from clockwork_amd.cache.manager import GroupLayout
from clockwork_amd.parts.base import EntryCache


def page_bytes(groups: list[GroupLayout], block_size: int, dtype: torch.dtype) -> int:
    """Bytes one page number occupies: its keys and values in every entry of every paged group
    (each group has a pool of ``num_blocks`` pages of its own)."""
    elem = torch.empty((), dtype=dtype).element_size()
    total = 0
    for group in groups:
        if group.is_kv:
            total += len(group.entries) * 2 * block_size * group.need.num_kv_heads * group.need.head_dim * elem
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
        self.kv: list[torch.Tensor] = []
        self.state: list[torch.Tensor] = []
        self._kv_index: dict[int, tuple[int, int]] = {}     # run entry -> (kv group, row)
        self._state_index: dict[int, tuple[int, int]] = {}  # run entry -> (state group, row)
        for group in groups:
            if group.is_kv:
                need = group.need
                shape = (len(group.entries), 2, num_blocks, block_size, need.num_kv_heads, need.head_dim)
                pool = torch.full(shape, fill, dtype=dtype, device=device)
                for row, entry in enumerate(group.entries):
                    self._kv_index[entry] = (len(self.kv), row)
                self.kv.append(pool)
            else:
                need = group.need
                shape = (len(group.entries), max_num_seqs + 1, *need.shape)
                pool = torch.zeros(shape, dtype=getattr(torch, need.dtype), device=device)
                if (pool[0, 0].numel() * pool.element_size()) % 4:
                    raise ValueError(f"a state of shape {tuple(need.shape)} {need.dtype} is not a whole number of "
                                     "32-bit words: the kernel that clears a fresh request's state takes words")
                for row, entry in enumerate(group.entries):
                    self._state_index[entry] = (len(self.state), row)
                self.state.append(pool)

    def bytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in self.kv + self.state)

    def kv_bytes_per_token(self) -> int:
        """Bytes of keys and values one cached token occupies, all groups and entries."""
        total = 0
        for pool in self.kv:
            total += pool.shape[0] * 2 * pool.shape[4] * pool.shape[5] * pool.element_size()
        return total

    def entry_cache(self, entry: int, source: int | None = None) -> EntryCache:
        """The cache of run entry ``entry``; with ``source`` the entry reads that entry's cache."""
        owner = entry if source is None else source
        if owner in self._kv_index:
            g, row = self._kv_index[owner]
            pool = self.kv[g]
            nkv, hd = pool.shape[4], pool.shape[5]
            return EntryCache(
                group=g,
                k=pool[row, 0].view(-1, nkv, hd),
                v=pool[row, 1].view(-1, nkv, hd),
                writes=source is None,
                block_size=self.block_size,
            )
        if owner in self._state_index:
            g, row = self._state_index[owner]
            return EntryCache(group=g, state=self.state[g][row], writes=source is None)
        return EntryCache(writes=False)

    def copy_pages(self, group: int, pairs: list[tuple[int, int]]) -> None:
        """Copy page src -> dst in every entry of the group (keys and values)."""
        if not pairs:
            return
        pool = self.kv[group]
        planes = pool.view(pool.shape[0] * 2, pool.shape[2], -1)
        ops.copy_pages(planes, torch.tensor(pairs, dtype=torch.int32, device=pool.device))

    def copy_state(self, src_slot: int, dst_slot: int) -> None:
        for pool in self.state:
            pool[:, dst_slot].copy_(pool[:, src_slot])

    def zero_fresh_state(self, state_slots: torch.Tensor, starts: torch.Tensor, n: int) -> None:
        """Clear the state of the step's requests that begin at position 0 (device int32 arrays of
        the step: each request's slot and first position). One kernel per state group; part of
        every step of a model with state, captured or not."""
        for pool in self.state:
            ops.zero_state_rows(pool, state_slots, starts, n)
