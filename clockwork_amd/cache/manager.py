"""The cache manager: pages of keys and values per layer group, block tables per request,
and slots for fixed-size per-request state.

Layer groups. Every run entry of a model that keeps a cache states its need
(:class:`KVPagesSpec` or :class:`StateSpec`). Entries with the same need form a
group. A key/value group has a page pool and, per request, a block table of its
own: a group that reads every earlier token keeps a request's pages until the
request ends; a group with a window gives pages back as soon as the window has
passed them, while the request still runs. A state group hands every live request
one slot. This architecture (Qwen2) has exactly one full key/value group and no
state group; the state slots exist so another mixer finds them.

What the reference's block manager decides is decided the same way here
(clockwork/kvcache/block_manager.py:6-101): admission needs the request's pages
plus a watermark of free ones, growth needs one page at a page boundary or for a
copy-on-write, a request that holds nothing cannot be freed twice.

This module is bookkeeping only and needs neither torch nor a GPU; device memory
is in ``clockwork_amd.cache.pools``.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Sequence

import numpy as np

from clockwork_amd.cache.allocator import OutOfPages, PagePool
from clockwork_amd.config.spec import KVPagesSpec, ModelSpec, PagedRowsSpec, StateSpec

NO_PAGE = -1


@dataclass(frozen=True)
class GroupLayout:
    """One layer group: which run entries it serves and what one of them stores."""

    index: int
    need: object            # KVPagesSpec / PagedRowsSpec (pages) or StateSpec (a slot)
    entries: tuple[int, ...]  # indices into ModelSpec.run that own a cache in this group

    @property
    def is_kv(self) -> bool:
        """Does the group keep rows per token in pages (keys and values, or planes of a mixer's own)?"""
        return isinstance(self.need, (KVPagesSpec, PagedRowsSpec))

    @property
    def window(self) -> Optional[int]:
        return self.need.window if self.is_kv else None


def plan_groups(needs: Sequence[Optional[object]]) -> list[GroupLayout]:
    """``needs[i]`` is what run entry ``i`` stores (None: nothing of its own).

    Groups come in order of first appearance, so a model's layout is stable."""
    order: list[tuple] = []
    members: dict[tuple, list[int]] = {}
    specs: dict[tuple, object] = {}
    for i, need in enumerate(needs):
        if need is None:
            continue
        if not isinstance(need, (KVPagesSpec, PagedRowsSpec, StateSpec)):
            raise TypeError(f"run entry {i}: a cache need must be KVPagesSpec, PagedRowsSpec or StateSpec, got {need!r}")
        key = need.group_key()
        if key not in members:
            order.append(key)
            members[key] = []
            specs[key] = need
        members[key].append(i)
    return [GroupLayout(g, specs[key], tuple(members[key])) for g, key in enumerate(order)]


@dataclass
class RequestPages:
    """What one live request holds."""

    tables: list[list[int]]              # per kv group: page of logical block b, NO_PAGE once released
    released: list[int]                  # per kv group: logical blocks below this index were given back
    state_slot: int = -1
    num_shared_prefix: int = 0           # leading logical blocks that came from the prefix cache
    epoch: int = 0                       # changes whenever an existing table entry changes (not on appends)


class CacheManager:
    def __init__(
        self,
        groups: Sequence[GroupLayout],
        block_size: int,
        num_blocks: int,
        max_num_seqs: int = 64,
        watermark: float = 0.0,
    ) -> None:
        if watermark < 0:
            raise ValueError(f"watermark must be non-negative, got {watermark}")
        self.groups = list(groups)
        self.kv_groups = [g for g in self.groups if g.is_kv]
        self.state_groups = [g for g in self.groups if not g.is_kv]
        self.block_size = block_size
        self.num_blocks = num_blocks
        self.pools = [PagePool(num_blocks, block_size) for _ in self.kv_groups]
        self.watermark_blocks = int(watermark * num_blocks)
        self.max_num_seqs = max_num_seqs
        self._free_slots = list(range(max_num_seqs - 1, -1, -1))
        # what a row that holds no request carries as its state slot: the pools' spare slot when
        # the model keeps state, else -1
        self.idle_state_slot = max_num_seqs if self.state_groups else -1
        self._requests: dict[str, RequestPages] = {}
        self._epochs = 0

    # ------------------------------------------------------------------ queries
    @property
    def supports_prefix_sharing(self) -> bool:
        """Cached pages are a function of the token prefix alone only when every group keeps
        all keys and nothing else is carried from token to token."""
        return bool(self.kv_groups) and not self.state_groups and all(g.window is None for g in self.kv_groups)

    def _next_epoch(self) -> int:
        self._epochs += 1
        return self._epochs

    def has(self, seq_id: str) -> bool:
        return seq_id in self._requests

    def record(self, seq_id: str) -> RequestPages:
        return self._requests[seq_id]

    def live_requests(self) -> list[str]:
        return list(self._requests)

    def num_free_blocks(self, group: int = 0) -> int:
        return self.pools[group].num_free if self.pools else 0

    def min_free_blocks(self) -> int:
        return min((p.num_free for p in self.pools), default=self.num_blocks)

    def block_table(self, seq_id: str, group: int = 0) -> list[int]:
        return self._requests[seq_id].tables[group]

    def state_slot(self, seq_id: str) -> int:
        return self._requests[seq_id].state_slot

    def _blocks_for(self, num_tokens: int) -> int:
        return -(-num_tokens // self.block_size)

    def _first_needed_block(self, g: int, computed: int) -> int:
        """Logical block of the oldest key the token at position ``computed`` reads in group g."""
        window = self.kv_groups[g].window
        if window is None:
            return 0
        return max(0, computed - window + 1) // self.block_size

    # ------------------------------------------------------------------ admission
    def _admission_extent(self, g: int, total_len: int, portion_end: int) -> int:
        # a full group reserves the whole request up front (the reference's arithmetic,
        # block_manager.py:25-40); a windowed group only what the first portion touches
        return total_len if self.kv_groups[g].window is None else portion_end

    def can_admit(self, total_len: int, portion_end: Optional[int] = None,
                  prefix_blocks: int = 0) -> bool:
        """Would a request of ``total_len`` tokens fit, leaving the watermark free?

        ``prefix_blocks`` leading blocks come from the prefix cache and cost nothing."""
        portion_end = total_len if portion_end is None else portion_end
        if self.state_groups and not self._free_slots:
            return False
        for g, pool in enumerate(self.pools):
            need = self._blocks_for(self._admission_extent(g, total_len, portion_end)) - prefix_blocks
            if pool.num_free - max(0, need) < self.watermark_blocks:
                return False
        return True

    def admit(self, seq_id: str, total_len: int, portion_end: Optional[int] = None,
              prefix: Sequence[tuple[int, ...]] = ()) -> RequestPages:
        """Take pages (and a state slot) for a new request. ``prefix`` holds, per leading
        block, the pages of every kv group that the prefix cache matched; the caller has
        already taken a hold on each of them for this request."""
        if seq_id in self._requests:
            raise ValueError(f"sequence {seq_id} already holds pages")
        portion_end = total_len if portion_end is None else portion_end
        if prefix and not self.supports_prefix_sharing:
            raise ValueError("this model's cache cannot share prefixes")
        needs = []
        for g, pool in enumerate(self.pools):
            need = max(0, self._blocks_for(self._admission_extent(g, total_len, portion_end)) - len(prefix))
            if need > pool.num_free:
                raise OutOfPages(f"layer group {g}: {need} pages wanted, {pool.num_free} free")
            needs.append(need)
        if self.state_groups and not self._free_slots:
            raise OutOfPages("no free state slot")
        tables = []
        for g, pool in enumerate(self.pools):
            tables.append([handle[g] for handle in prefix] + pool.take_many(needs[g]))
        rec = RequestPages(
            tables=tables,
            released=[0] * len(self.pools),
            state_slot=self._free_slots.pop() if self.state_groups else -1,
            num_shared_prefix=len(prefix),
            epoch=self._next_epoch(),
        )
        self._requests[seq_id] = rec
        return rec

    # ------------------------------------------------------------------ growth
    def _growth(self, rec: RequestPages, g: int, computed: int, upto: int) -> tuple[int, bool]:
        """(new pages, copy-on-write needed) for group g to back positions [computed, upto)."""
        table = rec.tables[g]
        new = max(0, self._blocks_for(upto) - len(table))
        cow = False
        logical = computed // self.block_size
        if logical < len(table) and table[logical] != NO_PAGE:
            cow = self.pools[g].is_shared(table[logical])
        return new, cow

    def _fits_as_is(self, rec: RequestPages, computed: int, upto: int) -> bool:
        """The common case of a decode step: the pages are there and the one written to is private."""
        size = self.block_size
        logical = computed // size
        for g, pool in enumerate(self.pools):
            table = rec.tables[g]
            if upto > len(table) * size:
                return False
            page = table[logical]
            if page != NO_PAGE and pool._holders[page] > 1:
                return False
        return True

    def can_extend(self, seq_id: str, computed: int, upto: int) -> bool:
        """Can the request write positions [computed, upto)? A page boundary needs a free page,
        a shared page under the write position needs one for its private copy
        (block_manager.py:44-54)."""
        rec = self._requests[seq_id]
        if self._fits_as_is(rec, computed, upto):
            return True
        for g, pool in enumerate(self.pools):
            new, cow = self._growth(rec, g, computed, upto)
            if new + (1 if cow else 0) > pool.num_free:
                return False
        return True

    def can_extend_all(self, spans) -> bool:
        """Can every one of these requests write its positions at once? ``spans``:
        ``(seq_id, computed, upto)`` each. (``can_extend`` answers for one request alone: three
        requests at a page's edge with two pages free can each, but not all.)"""
        need = [0] * len(self.pools)
        for seq_id, computed, upto in spans:
            rec = self._requests[seq_id]
            if self._fits_as_is(rec, computed, upto):
                continue
            for g in range(len(self.pools)):
                new, cow = self._growth(rec, g, computed, upto)
                need[g] += new + (1 if cow else 0)
        return all(n <= pool.num_free for n, pool in zip(need, self.pools))

    def extend(self, seq_id: str, computed: int, upto: int) -> list[tuple[int, int, int]]:
        """Back positions [computed, upto). Returns ``(group, src_page, dst_page)`` copies the
        caller must perform on the device before the step runs."""
        rec = self._requests[seq_id]
        if self._fits_as_is(rec, computed, upto):
            return []
        if not self.can_extend(seq_id, computed, upto):
            raise OutOfPages(f"sequence {seq_id}: no pages to grow to {upto} tokens")
        copies: list[tuple[int, int, int]] = []
        for g, pool in enumerate(self.pools):
            table = rec.tables[g]
            new, cow = self._growth(rec, g, computed, upto)
            if cow:
                logical = computed // self.block_size
                src, dst = pool.private_copy(table[logical])
                table[logical] = dst
                rec.epoch = self._next_epoch()
                copies.append((g, src, dst))
            table.extend(pool.take_many(new))
        return copies

    def release_behind_window(self, seq_id: str, computed: int) -> int:
        """After ``computed`` tokens are cached: give back pages no later token will read."""
        rec = self._requests[seq_id]
        given_back = 0
        for g, pool in enumerate(self.pools):
            if self.kv_groups[g].window is None:
                continue
            first = min(self._first_needed_block(g, computed), len(rec.tables[g]))
            for b in range(rec.released[g], first):
                page = rec.tables[g][b]
                if page != NO_PAGE:
                    pool.drop(page)
                    rec.tables[g][b] = NO_PAGE
                    rec.epoch = self._next_epoch()
                    given_back += 1
            rec.released[g] = max(rec.released[g], first)
        return given_back

    # ------------------------------------------------------------------ sharing and freeing
    def fork(self, parent_id: str, child_id: str) -> Optional[tuple[int, int]]:
        """The child shares every page of the parent (block_manager.py:77-83); state is not
        shared: the returned ``(src_slot, dst_slot)`` must be copied on the device."""
        if child_id in self._requests:
            raise ValueError(f"child {child_id} already has blocks")
        parent = self._requests[parent_id]
        if self.state_groups and not self._free_slots:
            raise OutOfPages("no free state slot")
        for g, pool in enumerate(self.pools):
            for page in parent.tables[g]:
                if page != NO_PAGE:
                    pool.share(page)
        slot = self._free_slots.pop() if self.state_groups else -1
        self._requests[child_id] = RequestPages(
            tables=[list(t) for t in parent.tables],
            released=list(parent.released),
            state_slot=slot,
            num_shared_prefix=parent.num_shared_prefix,
            epoch=self._next_epoch(),
        )
        return (parent.state_slot, slot) if self.state_groups else None

    def free(self, seq_id: str) -> None:
        rec = self._requests.pop(seq_id, None)
        if rec is None:
            raise ValueError(f"sequence {seq_id} holds no blocks (double free?)")
        for g, pool in enumerate(self.pools):
            pool.drop_many(page for page in rec.tables[g] if page != NO_PAGE)
        if rec.state_slot >= 0:
            self._free_slots.append(rec.state_slot)

    # holds taken and dropped on behalf of the prefix cache: one handle = one page per kv group
    def share_handle(self, handle: tuple[int, ...]) -> None:
        for pool, page in zip(self.pools, handle):
            pool.share(page)

    def drop_handle(self, handle: tuple[int, ...]) -> None:
        for pool, page in zip(self.pools, handle):
            pool.drop(page)

    def share_handles(self, handles: Sequence[tuple[int, ...]]) -> None:
        """``share_handle`` for many handles at once."""
        for g, pool in enumerate(self.pools):
            pool.share_many(handle[g] for handle in handles)

    def handles(self, seq_id: str, num_blocks: int) -> list[tuple[int, ...]]:
        rec = self._requests[seq_id]
        if any(len(t) < num_blocks for t in rec.tables):
            raise IndexError(f"sequence {seq_id} holds fewer than {num_blocks} blocks")
        return list(zip(*(t[:num_blocks] for t in rec.tables)))

    # ------------------------------------------------------------------ addressing
    def slot_mapping(self, seq_id: str, start: int, end: int, group: int = 0) -> list[int]:
        """Flat cache rows of positions [start, end): page * block_size + offset
        (block_manager.py:92-98)."""
        table = self._requests[seq_id].tables[group]
        size = self.block_size
        covered = len(table) * size
        if not 0 <= start <= end <= covered:
            raise ValueError(f"token range [{start}, {end}) outside covered range [0, {covered})")
        if end - start <= 8:  # a decoded token or two: not worth an array
            out = []
            for pos in range(start, end):
                page = table[pos // size]
                if page == NO_PAGE:
                    raise ValueError(f"position {pos} lies in a page that was given back")
                out.append(page * size + pos % size)
            return out
        pos = np.arange(start, end, dtype=np.int64)
        pages = np.asarray(table[start // size : (end - 1) // size + 1], dtype=np.int64)[pos // size - start // size]
        if (pages == NO_PAGE).any():
            raise ValueError(f"position {int(pos[pages == NO_PAGE][0])} lies in a page that was given back")
        return (pages * size + pos % size).tolist()

    def audit(self) -> None:
        """No page lost or held twice: per pool, holders' counts equal reference counts."""
        for g, pool in enumerate(self.pools):
            pool.audit()
        # requests alone cannot explain prefix-cache holds; callers add those (see tests)


def cache_needs_of(spec: ModelSpec, mixers: Sequence[object]) -> list[Optional[object]]:
    """Per run entry: the need of its layer's mixer, or None when it borrows another entry's cache."""
    needs: list[Optional[object]] = []
    for entry in spec.run:
        needs.append(None if entry.cache_from is not None else mixers[entry.layer].cache_need())
    return needs
