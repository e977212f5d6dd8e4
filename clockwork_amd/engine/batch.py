"""One step's batch: which request contributes which tokens, laid out for the kernels.

A step holds R requests; request r contributes q_len[r] >= 1 consecutive tokens
starting at position start[r]: a portion of a prompt, a whole prompt, or one decoded
token. All index arrays are packed into one pinned int32 buffer and go to the GPU
in a single copy; the kernels read device views of that buffer.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Sequence

import numpy as np
import torch


@dataclass
class StepEntry:
    """Next tokens of one request. ``want``: indices into ``tokens`` whose logits are asked for."""

    seq_id: str
    start: int
    tokens: Sequence[int]
    want: Sequence[int] = ()


class _Packer:
    def __init__(self) -> None:
        self.parts: list[np.ndarray] = []
        self.offsets: list[tuple[int, int]] = []
        self.size = 0

    def add(self, values) -> int:
        a = np.asarray(values, dtype=np.int32).reshape(-1)
        pad = (-self.size) % 4  # keep every array 16-byte aligned
        if pad:
            self.parts.append(np.zeros(pad, dtype=np.int32))
            self.size += pad
        self.offsets.append((self.size, a.size))
        self.parts.append(a)
        self.size += a.size
        return len(self.offsets) - 1

    def upload(self, device) -> list[torch.Tensor]:
        host = torch.empty(max(self.size, 1), dtype=torch.int32, pin_memory=True)
        if self.size:
            host.numpy()[: self.size] = np.concatenate(self.parts)
        dev = host.to(device, non_blocking=True)
        self._host = host  # keep the pinned buffer alive until the copy has run
        return [dev[o : o + n] for o, n in self.offsets]


class StepContext:
    """Everything a part may ask about the step. Built by :func:`build_context`."""

    def __init__(self) -> None:
        self.num_tokens = 0
        self.num_requests = 0
        self.num_logit_rows = 0
        self.device = None
        self.block_size = 0
        # device int32 tensors
        self.token_ids = None
        self.positions = None            # [T] what the parts read as positions (the embedding part may replace it)
        self.sequence_positions = None   # [T] each token's index in its request: start + i
        self.cu_q = None          # [R + 1]
        self.ctx_lens = None      # [R]  keys of each request once this step's tokens are cached
        self.starts = None        # [R]  position of each request's first token in this step
        self.state_slots = None   # [R]
        self.logit_rows = None    # [num_logit_rows] rows of the flat batch
        self.slots: list[torch.Tensor] = []         # per kv group [T]
        self.block_tables: list[torch.Tensor] = []  # per kv group [R, max_blocks]
        # host copies for planning
        self.h_q_lens: list[int] = []
        self.h_ctx_lens: list[int] = []
        self.h_starts: list[int] = []
        self.h_state_slots: list[int] = []
        self.seq_ids: list[str] = []
        self.plans: dict = {}     # what parts have planned for this step, under keys of their own
        self._pinned: list = []   # host buffers of the plans' uploads, alive as long as the step
        self.num_compute_units = 256
        self.products = None      # the engine's ops.ProductPolicy (None: the defaults)

    def upload(self, arrays) -> list:
        """int32 arrays to the device in one copy; returns a device view of each. For a part
        that plans its kernels' work items for this step (kept in ``plans``)."""
        packer = _Packer()
        for a in arrays:
            packer.add(a)
        views = packer.upload(self.device)
        self._pinned.append(packer)
        return views


def build_context(entries: Sequence[StepEntry], manager, device, vocab_size: int) -> StepContext:
    """Lay out ``entries`` (pages already reserved through ``manager``) as one batch."""
    ctx = StepContext()
    ctx.device = device
    ctx.block_size = manager.block_size
    tokens: list = []     # one array per entry
    positions: list = []
    cu = [0]
    logit_rows: list[int] = []
    state_slots: list[int] = []
    for e in entries:
        n = len(e.tokens)
        if n < 1:
            raise ValueError(f"request {e.seq_id}: a step entry needs at least one token")
        ids = np.asarray(e.tokens, dtype=np.int64)  # a long portion is checked as an array, not token by token
        if ids.shape != (n,) or ids.min() < 0 or ids.max() >= vocab_size:
            bad = next((t for t in e.tokens if not 0 <= int(t) < vocab_size), None)
            raise ValueError(f"request {e.seq_id}: token id {bad} outside the vocabulary [0, {vocab_size})")
        for w in e.want:
            if not 0 <= int(w) < n:
                raise ValueError(f"request {e.seq_id}: wanted index {w} outside its {n} tokens")
            logit_rows.append(cu[-1] + int(w))
        tokens.append(ids)
        positions.append(np.arange(e.start, e.start + n, dtype=np.int64))
        cu.append(cu[-1] + n)
        ctx.h_q_lens.append(n)
        ctx.h_starts.append(e.start)
        ctx.h_ctx_lens.append(e.start + n)
        ctx.seq_ids.append(e.seq_id)
        state_slots.append(manager.state_slot(e.seq_id))
    ctx.num_tokens = cu[-1]
    ctx.num_requests = len(entries)
    ctx.num_logit_rows = len(logit_rows)

    packer = _Packer()
    i_tok = packer.add(np.concatenate(tokens))
    i_pos = packer.add(np.concatenate(positions))
    i_cu = packer.add(cu)
    i_ctx = packer.add(ctx.h_ctx_lens)
    i_start = packer.add(ctx.h_starts)
    i_state = packer.add(state_slots)
    ctx.h_state_slots = state_slots
    i_rows = packer.add(logit_rows)
    group_idx = []
    for g in range(len(manager.kv_groups)):
        slots: list[int] = []
        width = max(1, max(-(-c // manager.block_size) for c in ctx.h_ctx_lens))
        table = np.full((len(entries), width), -1, dtype=np.int32)
        for r, e in enumerate(entries):
            slots += manager.slot_mapping(e.seq_id, e.start, e.start + len(e.tokens), g)
            row = manager.block_table(e.seq_id, g)[:width]
            table[r, : len(row)] = row
        group_idx.append((packer.add(slots), packer.add(table), width))
    views = packer.upload(device)
    ctx._packer = packer
    ctx.token_ids, ctx.positions, ctx.cu_q = views[i_tok], views[i_pos], views[i_cu]
    ctx.sequence_positions = ctx.positions
    ctx.ctx_lens, ctx.starts = views[i_ctx], views[i_start]
    ctx.state_slots, ctx.logit_rows = views[i_state], views[i_rows]
    for i_slots, i_table, width in group_idx:
        ctx.slots.append(views[i_slots])
        ctx.block_tables.append(views[i_table].view(len(entries), width))
    return ctx


class StaticDecodeBatch:
    """A decode-only batch with fixed shapes, for a captured HIP graph.

    ``size`` requests of one token each; every index array lives at a fixed device address and
    is refreshed by one host-to-device copy per step. Rows past the live requests are padding:
    token 0 at position 0, no cache slot (-1), no pages and the state pools' spare slot, so they
    write nothing that anyone reads and read nothing. ``key_capacity`` (the longest context the graph is planned for) only fixes how
    finely the attention kernel splits its keys.
    """

    def __init__(self, size: int, key_capacity: int, table_width: int, manager, device, prepare,
                 num_compute_units: int) -> None:
        self.size = size
        self.table_width = table_width
        n_groups = len(manager.kv_groups)
        self.block_size = manager.block_size
        # layout of the packed buffer
        offsets = {}
        at = 0

        def take(name, n):
            nonlocal at
            offsets[name] = (at, n)
            at += -(-n // 4) * 4

        for name in ("token_ids", "positions", "ctx_lens", "starts", "state_slots"):
            take(name, size)
        for g in range(n_groups):
            take(f"slots{g}", size)
            take(f"table{g}", size * table_width)
        self._offsets = offsets
        self.host = torch.zeros(at, dtype=torch.int32, pin_memory=True)
        self.device_buf = torch.zeros(at, dtype=torch.int32, device=device)
        self._np = self.host.numpy()

        def view(name):
            o, n = offsets[name]
            return self.device_buf[o : o + n]

        ctx = StepContext()
        ctx.device = device
        ctx.block_size = manager.block_size
        ctx.num_tokens = ctx.num_requests = ctx.num_logit_rows = size
        ctx.token_ids, ctx.positions = view("token_ids"), view("positions")
        ctx.sequence_positions = ctx.positions
        ctx.ctx_lens, ctx.starts, ctx.state_slots = view("ctx_lens"), view("starts"), view("state_slots")
        ctx.cu_q = torch.arange(size + 1, dtype=torch.int32, device=device)
        ctx.logit_rows = torch.arange(size, dtype=torch.int32, device=device)
        for g in range(n_groups):
            ctx.slots.append(view(f"slots{g}"))
            ctx.block_tables.append(view(f"table{g}").view(size, table_width))
        ctx.h_q_lens = [1] * size
        ctx.h_ctx_lens = [key_capacity] * size
        ctx.h_starts = [0] * size
        ctx.h_state_slots = [manager.idle_state_slot] * size
        ctx.seq_ids = [""] * size
        ctx.num_compute_units = num_compute_units
        prepare(ctx)  # the parts' work items are the same every step: made once, outside the graph
        self.ctx = ctx

    def fill(self, entries: Sequence[StepEntry], manager, upload: bool = True) -> None:
        """Write this step's indices into the pinned buffer and send them to the device.

        Block-table rows are kept from step to step: a row is rewritten only when another request
        moves into it or one of its entries changed (the request's ``epoch`` says so); otherwise
        just the newly taken pages are added. With ``upload`` off the buffer is only prepared (an
        entry's token may still be unknown: any placeholder): ``set_tokens`` and ``upload`` follow."""
        n = len(entries)
        size, width = self.size, self.table_width
        a = self._np
        bs = self.block_size
        sent = getattr(self, "_sent", None)
        if sent is not None:
            sent.synchronize()  # the copy of the step before must have read the buffer

        def region(name):
            o, cnt = self._offsets[name]
            return a[o : o + cnt]

        tok, pos = region("token_ids"), region("positions")
        ctx_lens, starts, state = region("ctx_lens"), region("starts"), region("state_slots")
        tok[n:] = 0
        pos[n:] = 0
        ctx_lens[n:] = 1
        starts[n:] = 0
        state[n:] = manager.idle_state_slot
        tok[:n] = [e.tokens[0] for e in entries]
        st = [e.start for e in entries]
        pos[:n] = st
        starts[:n] = st
        ctx_lens[:n] = pos[:n] + 1
        state[:n] = [manager.state_slot(e.seq_id) for e in entries]
        rows = getattr(self, "_rows", None)
        if rows is None:
            rows = self._rows = [[None, 0] for _ in range(size)]  # per row: epoch of the request in it, pages written
        for g in range(len(manager.kv_groups)):
            slots = region(f"slots{g}")
            table = region(f"table{g}").reshape(size, width)
            slots[n:] = -1
            for r, e in enumerate(entries):
                row = manager.block_table(e.seq_id, g)
                have = len(row)
                if have > width:
                    raise ValueError(f"request {e.seq_id} holds {have} pages, the graph was sized for {width}")
                state_r = rows[r]
                epoch = manager.record(e.seq_id).epoch
                if g > 0 or state_r[0] != epoch or state_r[1] > have:
                    table[r, :have] = row
                    table[r, have:] = -1
                elif state_r[1] < have:
                    table[r, state_r[1] : have] = row[state_r[1] :]
                if g == 0:
                    state_r[0], state_r[1] = epoch, have  # what group 0's row holds now: only it is written in pieces
                page = row[e.start // bs]
                if page < 0:
                    raise ValueError(f"request {e.seq_id}: position {e.start} lies in a page that was given back")
                slots[r] = page * bs + e.start % bs
            for r in range(n, size):
                if rows[r][0] is not None or g > 0:
                    table[r, :] = -1
                    if g == 0:
                        rows[r][0], rows[r][1] = None, 0
        self.ctx.seq_ids = [e.seq_id for e in entries] + [""] * (size - n)
        if upload:
            self.upload()

    def set_tokens(self, tokens: Sequence[int]) -> None:
        """The tokens of the entries that ``fill`` prepared."""
        o, _ = self._offsets["token_ids"]
        self._np[o : o + len(tokens)] = tokens

    def upload(self) -> None:
        self.device_buf.copy_(self.host, non_blocking=True)
        self._sent = torch.cuda.Event()
        self._sent.record()


class StaticPortionBatch:
    """One request's portion of up to ``num_tokens`` tokens with fixed shapes, for a captured HIP graph.

    A full-budget portion of a long prompt comes again and again with the same shape, and a short
    prompt fits the next larger of a few sizes: the index arrays live at fixed device addresses,
    refreshed by one host-to-device copy per step, and the attention work items are made once, for
    ``num_tokens`` tokens. A shorter portion leaves rows at the end that belong to no request:
    token 0, no cache slot, past the request's tokens as ``cu_q`` counts them, so no attention
    item computes them and nothing reads what the other kernels make of them. ``typical_start``
    is the position of a portion of the class of steps this batch serves (the parts choose their
    kernels' shapes by it, as they would for that step; any step's results are right under any
    such choice); ``wanted``: the logits of the portion's last token are made (else none).
    """

    def __init__(self, num_tokens: int, typical_start: int, wanted: bool, table_width: int, manager, device,
                 prepare, num_compute_units: int, vocab_size: int) -> None:
        self.num_tokens = n = num_tokens
        self.vocab_size = vocab_size
        self.table_width = table_width
        self.block_size = manager.block_size
        n_groups = len(manager.kv_groups)
        offsets = {}
        at = 0

        def take(name, count):
            nonlocal at
            offsets[name] = (at, count)
            at += -(-count // 4) * 4

        take("token_ids", n)
        take("positions", n)
        for name in ("ctx_lens", "starts", "state_slots", "logit_rows"):
            take(name, 1)
        take("cu_q", 2)
        for g in range(n_groups):
            take(f"slots{g}", n)
            take(f"table{g}", table_width)
        self._offsets = offsets
        self.host = torch.zeros(at, dtype=torch.int32, pin_memory=True)
        self.device_buf = torch.zeros(at, dtype=torch.int32, device=device)
        self._np = self.host.numpy()

        def view(name):
            o, count = offsets[name]
            return self.device_buf[o : o + count]

        ctx = StepContext()
        ctx.device = device
        ctx.block_size = manager.block_size
        ctx.num_tokens, ctx.num_requests, ctx.num_logit_rows = n, 1, int(wanted)
        ctx.token_ids, ctx.positions = view("token_ids"), view("positions")
        ctx.sequence_positions = ctx.positions
        ctx.ctx_lens, ctx.starts, ctx.state_slots = view("ctx_lens"), view("starts"), view("state_slots")
        ctx.cu_q = view("cu_q")
        ctx.logit_rows = view("logit_rows") if wanted else torch.empty(0, dtype=torch.int32, device=device)
        for g in range(n_groups):
            ctx.slots.append(view(f"slots{g}"))
            ctx.block_tables.append(view(f"table{g}").view(1, table_width))
        # what the parts' plans look at: the portion's length and where it starts
        ctx.h_q_lens = [n]
        ctx.h_ctx_lens = [typical_start + n]
        ctx.h_starts = [typical_start]
        ctx.h_state_slots = [manager.idle_state_slot]
        ctx.seq_ids = [""]
        ctx.num_compute_units = num_compute_units
        prepare(ctx)  # the parts' work items are the same every step: made once, outside the graph
        self.ctx = ctx

    def fill(self, entry: StepEntry, manager) -> None:
        """This step's indices into the pinned buffer, then to the device."""
        n, width = len(entry.tokens), self.table_width
        if not 0 < n <= self.num_tokens:
            raise ValueError(f"request {entry.seq_id}: {n} tokens for a batch of {self.num_tokens}")
        a = self._np
        sent = getattr(self, "_sent", None)
        if sent is not None:
            sent.synchronize()  # the copy of the step before must have read the buffer

        def region(name):
            o, count = self._offsets[name]
            return a[o : o + count]

        ids = np.asarray(entry.tokens, dtype=np.int64)
        if ids.shape != (n,) or ids.min() < 0 or ids.max() >= self.vocab_size:
            raise ValueError(f"request {entry.seq_id}: a token id outside the vocabulary [0, {self.vocab_size})")
        tok, pos = region("token_ids"), region("positions")
        tok[:n] = ids
        tok[n:] = 0
        pos[:n] = np.arange(entry.start, entry.start + n, dtype=np.int32)
        pos[n:] = 0
        region("ctx_lens")[0] = entry.start + n
        region("starts")[0] = entry.start
        region("state_slots")[0] = manager.state_slot(entry.seq_id)
        region("logit_rows")[0] = n - 1
        region("cu_q")[:] = (0, n)
        for g in range(len(manager.kv_groups)):
            slots = region(f"slots{g}")
            slots[:n] = manager.slot_mapping(entry.seq_id, entry.start, entry.start + n, g)
            slots[n:] = -1
            row = manager.block_table(entry.seq_id, g)
            if len(row) > width:
                raise ValueError(f"request {entry.seq_id} holds {len(row)} pages, the graph was sized for {width}")
            table = region(f"table{g}")
            table[: len(row)] = row
            table[len(row) :] = -1
        self.ctx.seq_ids = [entry.seq_id]
        self.device_buf.copy_(self.host, non_blocking=True)
        self._sent = torch.cuda.Event()
        self._sent.record()


class StaticMixedBatch:
    """Single decoded tokens of up to ``decoders`` requests beside one request's portion of up to
    ``portion`` tokens, with fixed shapes, for a captured HIP graph: the step that a short prompt
    makes when it arrives among decoding requests, which the host's launches would otherwise bound.

    Rows 0 .. decoders - 1 are the single tokens (request r in row r), the portion's tokens follow
    from row ``decoders``; the portion is request number ``decoders``. Rows and requests that a step
    does not fill are padding as in the two batches above: a single token 0 at position 0 of a
    request without pages, and rows behind the portion's tokens that ``cu_q`` leaves out. Logits
    are made for ``decoders + 1`` rows, which every step names anew (the wanted ones first, in the
    caller's order). ``key_capacity``: the longest context among the decoding requests the graph is
    planned for; ``typical_start``: where a portion of this class of steps begins.
    """

    def __init__(self, decoders: int, portion: int, key_capacity: int, typical_start: int, table_width: int,
                 manager, device, prepare, num_compute_units: int, vocab_size: int) -> None:
        self.decoders, self.portion = decoders, portion
        self.vocab_size = vocab_size
        self.table_width = table_width
        self.block_size = manager.block_size
        rows, requests = decoders + portion, decoders + 1
        n_groups = len(manager.kv_groups)
        offsets = {}
        at = 0

        def take(name, count):
            nonlocal at
            offsets[name] = (at, count)
            at += -(-count // 4) * 4

        take("token_ids", rows)
        take("positions", rows)
        for name in ("ctx_lens", "starts", "state_slots", "logit_rows"):
            take(name, requests)
        take("cu_q", requests + 1)
        for g in range(n_groups):
            take(f"slots{g}", rows)
            take(f"table{g}", requests * table_width)
        self._offsets = offsets
        self.host = torch.zeros(at, dtype=torch.int32, pin_memory=True)
        self.device_buf = torch.zeros(at, dtype=torch.int32, device=device)
        self._np = self.host.numpy()

        def view(name):
            o, count = offsets[name]
            return self.device_buf[o : o + count]

        ctx = StepContext()
        ctx.device = device
        ctx.block_size = manager.block_size
        ctx.num_tokens, ctx.num_requests, ctx.num_logit_rows = rows, requests, requests
        ctx.token_ids, ctx.positions = view("token_ids"), view("positions")
        ctx.sequence_positions = ctx.positions
        ctx.ctx_lens, ctx.starts, ctx.state_slots = view("ctx_lens"), view("starts"), view("state_slots")
        ctx.cu_q, ctx.logit_rows = view("cu_q"), view("logit_rows")
        for g in range(n_groups):
            ctx.slots.append(view(f"slots{g}"))
            ctx.block_tables.append(view(f"table{g}").view(requests, table_width))
        # what the parts' plans look at
        ctx.h_q_lens = [1] * decoders + [portion]
        ctx.h_ctx_lens = [key_capacity] * decoders + [typical_start + portion]
        ctx.h_starts = [0] * decoders + [typical_start]
        ctx.h_state_slots = [manager.idle_state_slot] * requests
        ctx.seq_ids = [""] * requests
        ctx.num_compute_units = num_compute_units
        prepare(ctx)  # the parts' work items are the same every step: made once, outside the graph
        self.ctx = ctx

    def row_of_portion(self, num_tokens: int) -> int:
        """The batch row of the last of the portion's ``num_tokens`` tokens."""
        return self.decoders + num_tokens - 1

    def fill(self, singles: Sequence[StepEntry], portion: StepEntry, manager, wanted_rows: Sequence[int]) -> None:
        """This step's indices into the pinned buffer, then to the device. ``singles``: the
        entries of one token each, in the order of their rows; ``portion``: the other entry;
        ``wanted_rows``: the batch rows whose logits the step makes first, in this order."""
        d, n = len(singles), len(portion.tokens)
        D, width, bs = self.decoders, self.table_width, self.block_size
        if d > D or not 0 < n <= self.portion:
            raise ValueError(f"{d} single tokens and a portion of {n} for a batch of {D} and {self.portion}")
        a = self._np
        sent = getattr(self, "_sent", None)
        if sent is not None:
            sent.synchronize()  # the copy of the step before must have read the buffer

        def region(name):
            o, count = self._offsets[name]
            return a[o : o + count]

        ids = np.asarray(portion.tokens, dtype=np.int64)
        if ids.shape != (n,) or ids.min() < 0 or ids.max() >= self.vocab_size:
            raise ValueError(f"request {portion.seq_id}: a token id outside the vocabulary [0, {self.vocab_size})")
        tok, pos = region("token_ids"), region("positions")
        ctx_lens, starts, state = region("ctx_lens"), region("starts"), region("state_slots")
        first = [e.start for e in singles]
        tok[:] = 0
        pos[:] = 0
        tok[:d] = [e.tokens[0] for e in singles]
        pos[:d] = first
        tok[D : D + n] = ids
        pos[D : D + n] = np.arange(portion.start, portion.start + n, dtype=np.int32)
        ctx_lens[:d] = pos[:d] + 1
        ctx_lens[d:D] = 1
        ctx_lens[D] = portion.start + n
        starts[:d] = first
        starts[d:D] = 0
        starts[D] = portion.start
        state[:d] = [manager.state_slot(e.seq_id) for e in singles]
        state[d:D] = manager.idle_state_slot
        state[D] = manager.state_slot(portion.seq_id)
        cu = region("cu_q")
        cu[: D + 1] = np.arange(D + 1, dtype=np.int32)
        cu[D + 1] = D + n
        if len(wanted_rows) > D + 1 or any(not 0 <= r < D + n for r in wanted_rows):
            raise ValueError("wanted rows outside the step's tokens")
        rows = region("logit_rows")
        rows[:] = 0
        rows[: len(wanted_rows)] = wanted_rows
        for g in range(len(manager.kv_groups)):
            slots = region(f"slots{g}")
            table = region(f"table{g}").reshape(D + 1, width)
            slots[:] = -1
            table[:] = -1
            for r, e in enumerate([*singles, portion]):
                row = manager.block_table(e.seq_id, g)
                if len(row) > width:
                    raise ValueError(f"request {e.seq_id} holds {len(row)} pages, the graph was sized for {width}")
                table[r if r < d else D, : len(row)] = row
            for r, e in enumerate(singles):
                page = manager.block_table(e.seq_id, g)[e.start // bs]
                if page < 0:
                    raise ValueError(f"request {e.seq_id}: position {e.start} lies in a page that was given back")
                slots[r] = page * bs + e.start % bs
            slots[D : D + n] = manager.slot_mapping(portion.seq_id, portion.start, portion.start + n, g)
        self.ctx.seq_ids = [e.seq_id for e in singles] + [""] * (D - d) + [portion.seq_id]
        self.device_buf.copy_(self.host, non_blocking=True)
        self._sent = torch.cuda.Event()
        self._sent.record()
