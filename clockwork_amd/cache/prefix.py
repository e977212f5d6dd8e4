"""Prefix cache: a trie over whole blocks of token ids that keeps the pages of finished prompts.

It offers what the reference's radix cache offers (clockwork/radix/cache.py:28-89,
clockwork/radix/tree.py:27-187) with a plainer structure: since matching is by
whole blocks anyway, every trie node is exactly one block (its key is the block's
tuple of token ids, its value the page handle), so there are no compressed edges
and nothing to split. Rules kept from the reference:

* a match never covers the whole sequence: at least one token is left to run
  (cache.py:43-48);
* a match takes one hold per matched block for the request and locks the deepest
  matched node; locked nodes and their ancestors are never evicted;
* insertion adopts (and takes a hold on) only blocks the trie did not have; for
  blocks it already has, the request keeps its own duplicate (cache.py:58-70);
* eviction removes unlocked leaves, least recently used first (tree.py:166-187).

A handle is a tuple with one page id per key/value group; holds are taken and
dropped through the ``share``/``drop`` callables (the cache manager's).
"""

from __future__ import annotations

import heapq
from dataclasses import dataclass, field
from typing import Callable, Optional, Sequence


@dataclass
class PrefixCacheStats:
    queries: int = 0
    hit_tokens: int = 0
    prompt_tokens: int = 0

    @property
    def hit_rate(self) -> float:
        return self.hit_tokens / self.prompt_tokens if self.prompt_tokens else 0.0


class _Node:
    __slots__ = ("parent", "key", "handle", "children", "stamp", "locks")

    def __init__(self, parent: Optional["_Node"], key: tuple, handle) -> None:
        self.parent = parent
        self.key = key
        self.handle = handle
        self.children: dict[tuple, _Node] = {}
        self.stamp = 0
        self.locks = 0


@dataclass
class PrefixMatch:
    num_tokens: int = 0
    handles: list = field(default_factory=list)
    node: Optional[_Node] = None  # the locked node; pass the match back to ``release``


class PrefixCache:
    def __init__(self, block_size: int, share: Callable, drop: Callable, enabled: bool = True,
                 share_many: Optional[Callable] = None) -> None:
        """``share(handle)`` / ``drop(handle)`` take and give back a hold on a block's pages;
        ``share_many(handles)``, when given, takes the holds of a whole match at once."""
        if block_size <= 0:
            raise ValueError(f"block_size must be positive, got {block_size}")
        self.block_size = block_size
        self.enabled = enabled
        self._share = share
        self._drop = drop
        self._share_many = share_many
        self.stats = PrefixCacheStats()
        self._root = _Node(None, (), None)
        self._tick = 0
        self._count = 0

    # ------------------------------------------------------------------ queries
    def num_blocks(self) -> int:
        return self._count

    def evictable_blocks(self) -> int:
        """Blocks that eviction could reach: not locked and with no locked descendant."""
        def walk(node: _Node) -> tuple[bool, int]:
            pinned = node.locks > 0
            total = 0
            for child in node.children.values():
                child_pinned, n = walk(child)
                pinned = pinned or child_pinned
                total += n
            if not pinned and node is not self._root:
                total += 1
            return pinned, total

        return walk(self._root)[1]

    def _blocks_of(self, token_ids: Sequence[int], n: int):
        bs = self.block_size
        for b in range(n):
            yield tuple(token_ids[b * bs : (b + 1) * bs])

    # ------------------------------------------------------------------ match / release
    def match(self, token_ids: Sequence[int]) -> PrefixMatch:
        self.stats.queries += 1
        self.stats.prompt_tokens += len(token_ids)
        if not self.enabled or not token_ids:
            return PrefixMatch()
        self._tick += 1
        limit = (len(token_ids) - 1) // self.block_size  # blocks strictly below the last token
        node = self._root
        handles = []
        for key in self._blocks_of(token_ids, limit):
            child = node.children.get(key)
            if child is None:
                break
            child.stamp = self._tick
            handles.append(child.handle)
            node = child
        if not handles:
            return PrefixMatch()
        if self._share_many is not None:
            self._share_many(handles)
        else:
            for handle in handles:
                self._share(handle)
        node.locks += 1
        matched = len(handles) * self.block_size
        self.stats.hit_tokens += matched
        return PrefixMatch(matched, handles, node)

    def release(self, match: PrefixMatch, drop_holds: bool = False) -> None:
        """Undo the lock of a match. With ``drop_holds`` also the holds taken for the request
        (an admission that did not go through); otherwise the request's pages are dropped by
        whoever frees the request."""
        if match.node is not None:
            match.node.locks -= 1
            match.node = None
        if drop_holds:
            for handle in match.handles:
                self._drop(handle)

    # ------------------------------------------------------------------ insert
    def insert(self, token_ids: Sequence[int], handles: Sequence) -> int:
        """Store the full blocks of ``token_ids`` with the pages ``handles``; returns how many
        blocks were new (and are now also held by the trie)."""
        if not self.enabled:
            return 0
        n = min(len(token_ids) // self.block_size, len(handles))
        if n == 0:
            return 0
        self._tick += 1
        node = self._root
        adopted = 0
        for b, key in enumerate(self._blocks_of(token_ids, n)):
            child = node.children.get(key)
            if child is None:
                child = _Node(node, key, handles[b])
                node.children[key] = child
                self._share(handles[b])
                self._count += 1
                adopted += 1
            child.stamp = self._tick
            node = child
        return adopted

    # ------------------------------------------------------------------ evict / reset
    def evict(self, num_blocks: int) -> int:
        """Remove up to ``num_blocks`` unlocked leaves, oldest first; a parent that becomes a leaf
        is a candidate at once. Returns the number removed."""
        if num_blocks <= 0:
            return 0
        heap: list[tuple[int, int, _Node]] = []
        stack = [self._root]
        serial = 0
        while stack:
            node = stack.pop()
            if node.children:
                stack.extend(node.children.values())
            elif node is not self._root and node.locks == 0:
                heap.append((node.stamp, serial, node))
                serial += 1
        heapq.heapify(heap)
        removed = 0
        while heap and removed < num_blocks:
            _, _, node = heapq.heappop(heap)
            parent = node.parent
            del parent.children[node.key]
            self._drop(node.handle)
            self._count -= 1
            removed += 1
            if parent is not self._root and not parent.children and parent.locks == 0:
                heapq.heappush(heap, (parent.stamp, serial, parent))
                serial += 1
        return removed

    def reset(self) -> None:
        stack = list(self._root.children.values())
        while stack:
            node = stack.pop()
            stack.extend(node.children.values())
            self._drop(node.handle)
        self._root = _Node(None, (), None)
        self._count = 0
        self.stats = PrefixCacheStats()
