"""Continuous batching: decode first, first-come-first-served admission, chunked prefill,
preemption by recompute.

The reference's decisions are kept (clockwork/scheduler/scheduler.py:34-204):

* running requests are served before anything is admitted, in order of arrival;
* when a running request cannot get the page it needs, the latest-arrived request
  that has not yet been served this step is preempted (the request itself if none is
  left): its pages go back, its progress is reset to zero, and it re-enters the
  waiting queue in front of every request that was never admitted;
* admission is strictly in queue order: a head that does not fit blocks the rest;
* admitting a request must leave the cache's watermark of pages free.

New here: a prompt no longer has to fit the token budget whole. A request
contributes ``min(remaining, budget left, max_prefill_chunk)`` tokens per step, so
running requests are either *prefilling* (more than one token still to run) or
*decoding* (exactly one). With ``enable_chunked_prefill`` off the reference's
behaviour returns: a prompt is admitted only whole (a request that was preempted and has
outgrown the budget by what it generated is the exception: it runs again in portions).

When pages run out: before a request is refused admission and before a running
request is preempted, idle blocks of the prefix cache are evicted, oldest first.
What then still does not fit waits (admission) or is preempted (running). A waiting
head that cannot be admitted although nothing runs and nothing can be evicted is an
error raised by the engine.
"""

from __future__ import annotations

from collections import deque
from dataclasses import dataclass, field
from typing import Optional

from clockwork_amd.cache.manager import CacheManager
from clockwork_amd.cache.prefix import PrefixCache, PrefixMatch
from clockwork_amd.config.engine import SchedulerConfig
from clockwork_amd.engine.sequence import Sequence, SequenceStatus


@dataclass
class ScheduledPortion:
    """``num_tokens`` tokens of ``seq`` starting at position ``start`` run in this step;
    ``samples`` is True when the portion reaches the sequence's end (a token is then drawn)."""

    seq: Sequence
    start: int
    num_tokens: int
    samples: bool


@dataclass
class SchedulerOutput:
    portions: list[ScheduledPortion] = field(default_factory=list)
    prefill_seqs: list[Sequence] = field(default_factory=list)  # sequences running more than one token
    decode_seqs: list[Sequence] = field(default_factory=list)   # sequences running exactly one
    preempted: list[Sequence] = field(default_factory=list)
    copies: list[tuple[int, int, int]] = field(default_factory=list)  # (group, src, dst) page copies
    num_batched_tokens: int = 0
    version: int = -1  # of the scheduler's queues, for an output made ahead of time (``schedule_ahead``)

    def is_empty(self) -> bool:
        return not (self.portions or self.preempted)


@dataclass
class SchedulerStats:
    num_waiting: int = 0
    num_running: int = 0
    num_preempted_total: int = 0
    num_scheduled_batches: int = 0
    total_prompt_tokens: int = 0
    total_cached_tokens: int = 0


class Scheduler:
    def __init__(self, cfg: SchedulerConfig, manager: CacheManager,
                 prefix_cache: Optional[PrefixCache] = None) -> None:
        self.cfg = cfg
        self.manager = manager
        self.prefix_cache = prefix_cache if (prefix_cache is not None and manager.supports_prefix_sharing) else None
        self.waiting: list[Sequence] = []
        self.running: list[Sequence] = []
        self.stats = SchedulerStats()
        self._matches: dict[str, PrefixMatch] = {}
        self._order: dict[str, int] = {}
        self._counter = 0
        # grows whenever a request arrives, leaves, is preempted or aborted: an output made ahead
        # of time is good only while it has not moved
        self.version = 0

    # ------------------------------------------------------------------ queue
    def _priority(self, seq: Sequence) -> tuple[float, int]:
        return (seq.arrival_time, self._order.get(seq.seq_id, 0))

    def add_seq(self, seq: Sequence) -> None:
        self._order[seq.seq_id] = self._counter
        self._counter += 1
        seq.status = SequenceStatus.WAITING
        self.waiting.append(seq)
        self.version += 1
        self._refresh()

    def has_unfinished(self) -> bool:
        return bool(self.waiting or self.running)

    def _refresh(self) -> None:
        self.stats.num_waiting = len(self.waiting)
        self.stats.num_running = len(self.running)

    # ------------------------------------------------------------------ giving back
    def _release(self, seq: Sequence) -> None:
        match = self._matches.pop(seq.seq_id, None)
        if match is not None and self.prefix_cache is not None:
            self.prefix_cache.release(match)  # the lock; the holds go with the pages below
        self.manager.free(seq.seq_id)

    def _preempt(self, seq: Sequence) -> None:
        """Take a running request's pages away. It keeps its tokens, loses its progress and waits
        again, ahead of every request that was never admitted and, among the preempted ones, in
        order of arrival (clockwork/scheduler/scheduler.py:79-96)."""
        self._release(seq)
        seq.reset_for_recompute()
        seq.num_cached_tokens = 0
        seq.status = SequenceStatus.PREEMPTED
        mine = self._priority(seq)
        ahead = 0
        for other in self.waiting:
            if other.status is not SequenceStatus.PREEMPTED or self._priority(other) > mine:
                break
            ahead += 1
        self.waiting.insert(ahead, seq)
        self.stats.num_preempted_total += 1
        self.version += 1

    def _evict_for(self, pages: int) -> bool:
        """Try to free ``pages`` pages from idle prefix-cache blocks; True if any went."""
        if self.prefix_cache is None or pages <= 0:
            return False
        return self.prefix_cache.evict(pages) > 0

    # ------------------------------------------------------------------ one step
    def _chunk(self, remaining: int, budget_left: int) -> int:
        n = min(remaining, budget_left)
        # the cap on a portion belongs to chunked prefill: without it a prompt runs whole, so a
        # cap would only keep every prompt longer than itself from ever running
        if self.cfg.max_prefill_chunk > 0 and self.cfg.enable_chunked_prefill:
            n = min(n, self.cfg.max_prefill_chunk)
        return n

    def _make_room(self, seq: Sequence, start: int, n: int, unserved: deque, out: SchedulerOutput) -> bool:
        """Free pages until ``seq`` can write positions [start, start + n): idle blocks of the
        prefix cache first; then running requests are preempted, the latest arrival among those
        not served yet in this step first, the request itself when no other is left
        (scheduler.py:98-113). False if ``seq`` itself had to go."""
        while not self.manager.can_extend(seq.seq_id, start, start + n):
            if self._evict_for(1):
                continue
            victim = unserved.pop() if unserved else seq
            self._preempt(victim)
            out.preempted.append(victim)
            if victim is seq:
                return False
        return True

    def _whole_only(self, seq: Sequence, remaining: int) -> bool:
        """Without chunked prefill a prompt runs whole or not at all (the reference's rule). A
        request that is run again after a preemption has grown by what it generated and may no
        longer fit the token budget: that one runs in portions, or it could never go on."""
        if self.cfg.enable_chunked_prefill:
            return False
        return not (seq.output_token_ids and remaining > self.cfg.max_num_batched_tokens)

    def _serve_running(self, out: SchedulerOutput) -> None:
        """Every running request, in order of arrival, gets its next tokens: one if it decodes
        (always served), else a portion of what it still has to run, as the budget allows."""
        unserved = deque(sorted(self.running, key=self._priority))
        budget = self.cfg.max_num_batched_tokens
        kept: list[Sequence] = []
        while unserved:
            seq = unserved.popleft()
            remaining = seq.num_uncomputed_tokens()
            n = 1 if remaining == 1 else self._chunk(remaining, budget - out.num_batched_tokens)
            if remaining > 1 and n < remaining and self._whole_only(seq, remaining):
                n = 0  # a prompt runs whole or not at all
            if n <= 0:
                kept.append(seq)  # stays running, contributes nothing this step
                continue
            start = seq.num_computed_tokens
            if not self._make_room(seq, start, n, unserved, out):
                continue
            out.copies += self.manager.extend(seq.seq_id, start, start + n)
            kept.append(seq)
            self._emit(out, seq, start, n)
        self.running = kept

    def _emit(self, out: SchedulerOutput, seq: Sequence, start: int, n: int, admitted: bool = False) -> None:
        samples = start + n == len(seq)
        out.portions.append(ScheduledPortion(seq, start, n, samples))
        decoding = seq.num_uncomputed_tokens() == 1 and not admitted
        (out.decode_seqs if decoding else out.prefill_seqs).append(seq)
        out.num_batched_tokens += n

    def _try_admit(self, seq: Sequence, out: SchedulerOutput) -> bool:
        match = PrefixMatch()
        if self.prefix_cache is not None:
            match = self.prefix_cache.match(seq.token_ids())
        cached = match.num_tokens
        remaining = len(seq) - cached
        budget_left = self.cfg.max_num_batched_tokens - out.num_batched_tokens
        n = self._chunk(remaining, budget_left)
        if n < remaining and self._whole_only(seq, remaining):
            n = 0
        fits = n > 0
        if fits:
            prefix_blocks = len(match.handles)
            if not self.manager.can_admit(len(seq), cached + n, prefix_blocks):
                # idle cached blocks are worth less than a waiting request
                need = -(-len(seq) // self.manager.block_size) - prefix_blocks
                short = need + self.manager.watermark_blocks - self.manager.min_free_blocks()
                self._evict_for(short)
                fits = self.manager.can_admit(len(seq), cached + n, prefix_blocks)
        if not fits:
            if self.prefix_cache is not None:
                self.prefix_cache.release(match, drop_holds=True)  # scheduler.py:132-140
            return False
        self.manager.admit(seq.seq_id, len(seq), cached + n, prefix=match.handles)
        if match.node is not None:
            self._matches[seq.seq_id] = match
        seq.num_cached_tokens = cached
        seq.num_computed_tokens = cached
        seq.status = SequenceStatus.RUNNING
        self.stats.total_prompt_tokens += len(seq)
        self.stats.total_cached_tokens += cached
        out.copies += self.manager.extend(seq.seq_id, cached, cached + n)
        self._emit(out, seq, cached, n, admitted=True)
        return True

    def schedule(self) -> SchedulerOutput:
        out = SchedulerOutput()
        self._serve_running(out)
        # the head of the queue or nobody: a request that does not fit holds back those behind it
        while (self.waiting and len(self.running) < self.cfg.max_num_seqs
               and self._try_admit(self.waiting[0], out)):
            self.running.append(self.waiting.pop(0))
        if not out.is_empty():
            self.stats.num_scheduled_batches += 1
        self._refresh()
        return out

    # ------------------------------------------------------------------ one step ahead
    def schedule_ahead(self, prev: SchedulerOutput, max_len: Optional[int] = None) -> Optional[SchedulerOutput]:
        """The step after ``prev``, decided while ``prev`` still runs on the GPU and its tokens
        are unknown, for the common case that nothing changes: nobody waits, every running
        request decoded one token in ``prev`` and none of them ends by length (``max_tokens``, the
        model length, ``max_len`` if the caller has a tighter one) with that token.
        The pages of the next positions are taken now; nothing is evicted or preempted ahead of
        time. Returns None when the ordinary ``schedule`` has to decide. The caller may use the
        result only if ``version`` still equals the scheduler's when the tokens have arrived (no
        request stopped, arrived or was aborted), and then calls ``commit_ahead``; a result
        that is dropped leaves the pages with their requests, which ask for them again anyway."""
        if self.waiting or prev.preempted or not prev.portions or len(prev.portions) != len(self.running):
            return None
        limit = self.cfg.max_model_len if max_len is None else min(self.cfg.max_model_len, max_len)
        for p in prev.portions:
            seq = p.seq
            if p.num_tokens != 1 or not p.samples or seq.status is not SequenceStatus.RUNNING:
                return None
            if (len(seq.output_token_ids) + 1 >= seq.sampling_params.max_tokens
                    or len(seq) + 1 >= limit):
                return None  # its last token is being made right now
        # all of them together: pages that are there for each alone may not be there for all
        if not self.manager.can_extend_all([(p.seq.seq_id, p.start + 1, p.start + 2) for p in prev.portions]):
            return None
        out = SchedulerOutput(version=self.version)
        for p in prev.portions:
            out.copies += self.manager.extend(p.seq.seq_id, p.start + 1, p.start + 2)
            out.portions.append(ScheduledPortion(p.seq, p.start + 1, 1, True))
            out.decode_seqs.append(p.seq)
            out.num_batched_tokens += 1
        return out

    def commit_ahead(self, out: SchedulerOutput) -> None:
        """``out`` of ``schedule_ahead`` is run as this step's schedule."""
        if out.version != self.version:
            raise RuntimeError("the schedule made ahead of time is out of date")
        self.stats.num_scheduled_batches += 1

    # ------------------------------------------------------------------ finishing
    def free_finished(self) -> None:
        for seq in self.running:
            if seq.is_finished():
                self._release(seq)
                self._order.pop(seq.seq_id, None)
                self.version += 1
        self.running = [seq for seq in self.running if not seq.is_finished()]
        self._refresh()

    def abort(self, seq_id: str) -> None:
        """Waiting and preempted requests hold nothing; a running one gives its pages back.
        An unknown id is ignored (scheduler.py:180-197)."""
        for queue, holds in ((self.waiting, False), (self.running, True)):
            for i, seq in enumerate(queue):
                if seq.seq_id == seq_id:
                    if holds:
                        self._release(seq)
                    queue.pop(i)
                    seq.status = SequenceStatus.FINISHED_ABORTED
                    self._order.pop(seq_id, None)
                    self.version += 1
                    self._refresh()
                    return
