"""The step function: run a batch of (request, its next tokens) from the cache, return logits.

``ModelRunner`` owns the model, the cache manager and the device pools. ``step`` takes
any mix of prompt portions and single decoded tokens, runs exactly the tokens it is
given as one flat batch and returns float32 logits at the wanted places. It samples
nothing: sampling sits above (``clockwork_amd.sampling``), so a replay tool can call
the step raw. The reference's runner ran one forward per prompt and one for all decode
tokens (clockwork/engine/model_runner.py:48-132); here they are one batch.
"""

from __future__ import annotations

import contextlib
import gc
from typing import Optional, Sequence

import torch

from clockwork_amd import ops
from clockwork_amd.cache.manager import CacheManager, cache_needs_of, plan_groups
from clockwork_amd.cache.pools import CachePools, pages_that_fit
from clockwork_amd.config.engine import EngineConfig
from clockwork_amd.engine.graph_nodes import node_kinds, only_kernels
from clockwork_amd.engine.batch import (
    StaticDecodeBatch,
    StaticMixedBatch,
    StaticPortionBatch,
    StepEntry,
    build_context,
)
from clockwork_amd.parts.model import DecoderModel
from clockwork_amd.registry import resolve_architecture
from clockwork_amd.weights.loader import load_parameters, read_config_json
from clockwork_amd.weights.random_init import RandomSource


# padded batch sizes a decode graph is captured for, and the step in which the planned context grows
GRAPH_BATCH_SIZES = (1, 2, 4, 8, 16, 24, 32, 48, 64, 96, 128, 192, 256)
GRAPH_KEY_BUCKET = 512
# a step that is one request's portion replays a graph captured for the token budget or for the
# next of these sizes (a step of 65 to 500 tokens is otherwise bound by the host's launches)
PORTION_GRAPH_SIZES = (16, 32, 64, 128, 256, 384, 512)
# the rows that the narrow products take in one, two or four tiles of tokens: a step of single
# tokens beside a short portion is padded to the next of these in all, if it fits one
NARROW_STEP_ROWS = (16, 32, 64)
# captured graphs kept at a time (each holds index buffers of its own): the least recently
# replayed one goes when another shape is captured beyond this many
GRAPH_LIMIT = 48


@contextlib.contextmanager
def capturing(graph: "torch.cuda.CUDAGraph", pool):
    """Capture the launches made inside into ``graph``. The cyclic garbage collector is off
    meanwhile: if it ran in the middle of a capture and found an unreachable runner, destroying
    that runner's captured graphs and device memory would be HIP calls that a capturing stream
    does not permit, and the error they raise inside a destructor ends the process."""
    was_enabled = gc.isenabled()
    gc.disable()
    try:
        with torch.cuda.graph(graph, pool=pool):
            yield
    finally:
        if was_enabled:
            gc.enable()


def require_gpu() -> torch.device:
    if not torch.cuda.is_available():
        raise RuntimeError(
            "clockwork_amd runs on an AMD GPU through its HIP kernels only: no GPU is visible "
            "(torch.cuda.is_available() is False) and there is no CPU path"
        )
    return torch.device("cuda", torch.cuda.current_device())


class ModelRunner:
    # the step of few rows that a tuning start-up runs for all of them
    FEW_ROWS_SAMPLE = 8

    def __init__(self, cfg: EngineConfig, weight_source=None, config_dict: Optional[dict] = None,
                 cache_fill: float = 0.0, use_graphs: bool = True) -> None:
        self.cfg = cfg
        if cfg.model.device not in ("cuda", "cuda:0", "gpu"):
            raise ValueError(f"device {cfg.model.device!r}: this engine runs on the GPU only")
        self.device = require_gpu()
        self.dtype = cfg.model.torch_dtype()
        # how this engine runs its large bfloat16 products (its own: another engine in the process
        # has another); the parts find it in every step's context
        self.products = ops.ProductPolicy(hip_products=cfg.model.hip_products)
        self.config_dict = config_dict if config_dict is not None else read_config_json(cfg.model.model)
        self.arch = resolve_architecture(self.config_dict)
        self.model_config = self.arch.parse_config(self.config_dict)
        self.spec = self.arch.build_spec(self.model_config)
        self.model = DecoderModel(self.spec)
        ops.preload(self.model.kernel_libraries(), tiled_products=cfg.model.hip_products or self.dtype == torch.bfloat16)
        plan = self.arch.weight_plan(self.model_config, self.spec)
        if weight_source is None and cfg.model.weights != "checkpoint":
            # a model without a checkpoint (clockwork/engine/loader.py:82-103 builds its tiny
            # models from a seed): the tensors a checkpoint would hold, drawn from the seed
            drawn_on = self.device if cfg.model.weights == "random_device" else "cpu"
            weight_source = RandomSource(plan, self.model.param_specs(), cfg.model.weight_seed, device=drawn_on)
        params = load_parameters(
            cfg.model.model, plan, self.model.param_specs(), self.dtype, self.device, source=weight_source
        )
        self.model.bind(params, self.device, self.dtype)

        groups = plan_groups(cache_needs_of(self.spec, self.model.mixers()))
        num_blocks = cfg.cache.num_blocks
        if num_blocks <= 0:
            # left open: what fits beside the weights, up to what the scheduler can ever use
            most = 2 * cfg.scheduler.max_num_seqs * -(-cfg.model.max_model_len // cfg.cache.block_size)
            num_blocks = pages_that_fit(groups, cfg.cache.block_size, self.dtype,
                                        torch.cuda.mem_get_info(self.device)[0], cfg.cache.memory_fraction, most)
        self.num_blocks = num_blocks
        self.manager = CacheManager(
            groups,
            block_size=cfg.cache.block_size,
            num_blocks=num_blocks,
            max_num_seqs=cfg.scheduler.max_num_seqs,
            watermark=cfg.cache.watermark,
        )
        self.pools = CachePools(
            groups, cfg.cache.block_size, num_blocks, cfg.scheduler.max_num_seqs,
            self.dtype, self.device, fill=cache_fill,
        )
        self.caches = [self.pools.entry_cache(i, e.cache_from) for i, e in enumerate(self.spec.run)]
        self.num_compute_units = torch.cuda.get_device_properties(self.device).multi_processor_count
        # decode-only steps replay captured HIP graphs: one per (padded batch size, context bucket)
        self.use_graphs = use_graphs and self.model.graph_safe()
        self._graphs: dict = {}
        self.graph_nodes: dict = {}  # per captured shape: how many nodes of each kind its graph held
        self._graph_pool = None
        self._table_width = -(-cfg.model.max_model_len // cfg.cache.block_size)

    # ------------------------------------------------------------------ pages
    def reserve(self, seq_id: str, start: int, num_tokens: int, total_len: Optional[int] = None) -> None:
        """Make sure positions [start, start + num_tokens) of the request are backed by pages;
        a new request is admitted (``total_len``: pages to set aside for it in groups that keep
        every key), a known one grows. Copy-on-write copies are done here."""
        end = start + num_tokens
        if not self.manager.has(seq_id):
            if start != 0:
                raise ValueError(f"request {seq_id} is unknown but starts at position {start}")
            self.manager.admit(seq_id, max(total_len or end, end), end)
        copies = self.manager.extend(seq_id, start, end)
        self.apply_copies(copies)

    def apply_copies(self, copies: Sequence[tuple[int, int, int]]) -> None:
        by_group: dict[int, list[tuple[int, int]]] = {}
        for g, src, dst in copies:
            by_group.setdefault(g, []).append((src, dst))
        for g, pairs in by_group.items():
            self.pools.copy_pages(g, pairs)

    def share_prefix(self, seq_id: str, source_id: str, num_tokens: int) -> None:
        """Admit ``seq_id`` as a request whose first ``num_tokens`` tokens are the ones the live
        request ``source_id`` has cached: it holds the same pages (what a prefix-cache hit gives
        a request) and goes on at position ``num_tokens``. A last page that is only partly
        covered is shared too; whoever writes to it first gets a copy of its own (``reserve``)."""
        if self.manager.has(seq_id):
            raise ValueError(f"request {seq_id} holds pages already")
        blocks = -(-num_tokens // self.manager.block_size)
        if num_tokens < 1 or any(blocks > len(self.manager.block_table(source_id, g))
                                 for g in range(len(self.manager.kv_groups))):
            raise ValueError(f"request {source_id} does not hold {num_tokens} tokens to share")
        handles = self.manager.handles(source_id, blocks)
        self.manager.admit(seq_id, num_tokens, prefix=handles)  # refuses models whose cache cannot be shared
        for handle in handles:
            self.manager.share_handle(handle)

    def fork(self, parent_id: str, child_id: str) -> None:
        """``child_id`` starts as a copy of the live request ``parent_id``: every page shared
        (copied when either writes into it), fixed-size state copied now."""
        slots = self.manager.fork(parent_id, child_id)
        if slots is not None:
            self.pools.copy_state(*slots)

    def release(self, seq_id: str) -> None:
        if self.manager.has(seq_id):
            self.manager.free(seq_id)

    # ------------------------------------------------------------------ library products
    @torch.no_grad()
    def tune_products(self, token_counts: Sequence[int]) -> list[int]:
        """Let the matrix library choose its fastest kernel for the products of steps with these
        token counts: each count runs once as a throwaway request while tuning is on. Counts the
        hand-written narrow products serve (but for one step of 8 tokens, which stands for all
        steps of few rows: the engine times its own choices for them on it, such as into how many
        parts over K a product is summed), float32 models (no library product) and counts that the
        cache cannot hold are skipped. Returns the counts that ran."""
        done: list[int] = []
        if self.dtype != torch.bfloat16:
            return done
        limit = min(self.cfg.model.max_model_len, self._table_width * self.manager.block_size)
        counts = {int(c) for c in token_counts}
        if any(c <= ops.SKINNY_MAX_ROWS for c in counts):
            counts.add(self.FEW_ROWS_SAMPLE)
        for n in sorted(counts, reverse=True):
            if (n <= ops.SKINNY_MAX_ROWS and n != self.FEW_ROWS_SAMPLE) or n > limit:
                continue
            seq_id = "__tune_products__"
            if not self.manager.can_admit(n, n):
                continue
            self.reserve(seq_id, 0, n, total_len=n)
            try:
                with ops.library_tuning(self.products):
                    self.step([StepEntry(seq_id, 0, [0] * n, [n - 1])])
                torch.cuda.synchronize()
                done.append(n)
            finally:
                self.release(seq_id)
        return done

    # ------------------------------------------------------------------ decode steps as graphs
    def _graph_step(self, entries: Sequence[StepEntry]):
        """Replay the captured graph for this batch shape. The first step of a shape runs eagerly
        (it loads and initialises whatever is still lazy), the second is captured, later ones
        replay. Returns NotImplemented when the step has to take the ordinary path."""
        n = len(entries)
        size = next(b for b in GRAPH_BATCH_SIZES if b >= n)
        longest = max(e.start + 1 for e in entries)
        if longest > self._table_width * self.manager.block_size:
            return NotImplemented
        capacity = GRAPH_KEY_BUCKET * -(-longest // GRAPH_KEY_BUCKET)
        key = (size, capacity)
        state = self._graphs.get(key)
        if state is None:
            self._graphs[key] = "seen"
            return NotImplemented
        if state == "eager":
            return NotImplemented
        for e in entries:
            if not 0 <= int(e.tokens[0]) < self.spec.vocab_size:
                raise ValueError(f"request {e.seq_id}: token id {e.tokens[0]} outside the vocabulary")
            if any(w != 0 for w in e.want):
                raise ValueError(f"request {e.seq_id}: wanted index outside its 1 token")
        if state == "seen":
            batch = StaticDecodeBatch(size, capacity, self._table_width, self.manager, self.device,
                                      self.model.prepare, self.num_compute_units)
            batch.fill(entries, self.manager)
            torch.cuda.synchronize()
            state = self._capture(key, batch)
            if state is None:
                return NotImplemented
        self._graphs[key] = self._graphs.pop(key)  # most recently used last
        batch, graph, out = state
        batch.fill(entries, self.manager)
        graph.replay()
        for e in entries:
            self.manager.release_behind_window(e.seq_id, e.start + 1)
        rows = [r for r, e in enumerate(entries) if len(e.want)]
        if not rows:
            return None
        if len(rows) == n:
            return out[:n]
        return out[torch.tensor(rows, device=self.device)]

    def _portion_graph_step(self, entry: StepEntry):
        """A step that is one portion of one request, of the token budget (what a long prompt's
        prefill is made of) or of up to 512 tokens (a short prompt, the end of a long one), replays
        a captured graph as the decode steps do, padded to the next of a few sizes: the first step
        of a shape runs eagerly, the second is captured.
        Returns NotImplemented when the step has to take the ordinary path."""
        n = len(entry.tokens)
        want = [int(w) for w in entry.want]
        if want not in ([], [n - 1]) or entry.start + n > self._table_width * self.manager.block_size:
            return NotImplemented
        budget = self.cfg.scheduler.max_num_batched_tokens
        size = n if n == budget else next((b for b in PORTION_GRAPH_SIZES if b >= n), None)
        if size is None:
            return NotImplemented
        # the parts may run other kernels for a portion behind many cached keys than for an early
        # one: a graph serves the portions of its own class (judged for the padded size)
        key = ("portion", size, self.model.shape_class([size], [entry.start + size]), bool(want))
        state = self._graphs.get(key)
        if state is None:
            self._graphs[key] = "seen"
            return NotImplemented
        if state == "eager":
            return NotImplemented
        if state == "seen":
            batch = StaticPortionBatch(size, entry.start, bool(want), self._table_width, self.manager, self.device,
                                       self.model.prepare, self.num_compute_units, self.spec.vocab_size)
            batch.fill(entry, self.manager)
            torch.cuda.synchronize()
            state = self._capture(key, batch)
            if state is None:
                return NotImplemented
        self._graphs[key] = self._graphs.pop(key)  # most recently used last
        batch, graph, out = state
        batch.fill(entry, self.manager)
        graph.replay()
        self.manager.release_behind_window(entry.seq_id, entry.start + n)
        return out if want else None

    def _mixed_graph_step(self, entries: Sequence[StepEntry]):
        """A step of single decoded tokens beside one request's portion of up to 512 tokens (a
        short prompt that arrives among decoding requests, or a portion of a longer one) replays a
        captured graph as well: padded to the next batch size and the next portion size (so that
        a step of up to 64 rows in all keeps to the 16, 32 or 64 rows of the narrow products), per
        context bucket of the decoding requests and class of the portion. The first step of a
        shape runs eagerly, the second is captured. Returns NotImplemented when the step has to
        take the ordinary path."""
        where = [i for i, e in enumerate(entries) if len(e.tokens) > 1]
        if len(where) != 1:
            return NotImplemented
        portion = entries[where[0]]
        singles = [e for e in entries if e is not portion]
        n, d = len(portion.tokens), len(singles)
        want = [int(w) for w in portion.want]
        decoders = next(b for b in GRAPH_BATCH_SIZES if b >= d)
        rows = next((t for t in NARROW_STEP_ROWS if decoders + n <= t), None)
        size = rows - decoders if rows else next((b for b in PORTION_GRAPH_SIZES if b >= max(n, NARROW_STEP_ROWS[-1])), None)
        limit = self._table_width * self.manager.block_size
        if size is None or want not in ([], [n - 1]) or portion.start + n > limit:
            return NotImplemented
        longest = max(e.start + 1 for e in singles)
        if longest > limit:
            return NotImplemented
        # the decoding requests' context in powers of two (it only sets how finely their keys are
        # split): with two other sizes in the key, finer steps would make too many shapes
        capacity = GRAPH_KEY_BUCKET
        while capacity < longest:
            capacity *= 2
        shape = self.model.shape_class([1] * decoders + [size], [capacity] * decoders + [portion.start + size])
        key = ("mixed", decoders, size, capacity, shape)
        state = self._graphs.get(key)
        if state is None:
            self._graphs[key] = "seen"
            return NotImplemented
        if state == "eager":
            return NotImplemented
        for e in singles:
            if not 0 <= int(e.tokens[0]) < self.spec.vocab_size:
                raise ValueError(f"request {e.seq_id}: token id {e.tokens[0]} outside the vocabulary")
            if any(w != 0 for w in e.want):
                raise ValueError(f"request {e.seq_id}: wanted index outside its 1 token")
        # the rows whose logits are wanted, in the order of the entries: single token r is row r of
        # the batch, the portion's tokens follow the (padded) single tokens
        row_of = {id(e): r for r, e in enumerate(singles)}
        row_of[id(portion)] = decoders + n - 1
        wanted_rows = [row_of[id(e)] for e in entries if len(e.want)]
        if state == "seen":
            batch = StaticMixedBatch(decoders, size, capacity, portion.start, self._table_width, self.manager,
                                     self.device, self.model.prepare, self.num_compute_units, self.spec.vocab_size)
            batch.fill(singles, portion, self.manager, wanted_rows)
            torch.cuda.synchronize()
            state = self._capture(key, batch)
            if state is None:
                return NotImplemented
        self._graphs[key] = self._graphs.pop(key)  # most recently used last
        batch, graph, out = state
        batch.fill(singles, portion, self.manager, wanted_rows)
        graph.replay()
        for e in entries:
            self.manager.release_behind_window(e.seq_id, e.start + len(e.tokens))
        return out[: len(wanted_rows)] if wanted_rows else None

    def _capture(self, key, batch):
        """Capture the model's step on ``batch`` (filled, its copy done) as the graph of ``key``.
        A graph that holds anything but kernel nodes is not kept (a library product may record a
        memset of its workspace, and such nodes have replayed wrongly): its shape is marked to
        run eagerly from now on and None is returned."""
        graph = torch.cuda.CUDAGraph(keep_graph=True)
        with capturing(graph, self._graph_pool):
            out = self._forward(batch.ctx)
        kinds = node_kinds(graph)
        self.graph_nodes[key] = dict(kinds)
        if not only_kernels(kinds):
            torch.cuda.synchronize()
            graph.reset()
            self._graphs[key] = "eager"
            return None
        graph.instantiate()
        if self._graph_pool is None:
            self._graph_pool = graph.pool()
        self._graphs.pop(key, None)  # the newest entry: another one goes when there are too many
        state = self._graphs[key] = (batch, graph, out)
        self._drop_old_graphs()
        return state

    def _drop_old_graphs(self) -> None:
        captured = [k for k, v in self._graphs.items() if isinstance(v, tuple)]
        if len(captured) <= GRAPH_LIMIT:
            return
        torch.cuda.synchronize()  # none of them may still be running
        for k in captured[: len(captured) - GRAPH_LIMIT]:
            del self._graphs[k]

    def prepare_decode(self, positions: Sequence[tuple[str, int]]):
        """Get a decode-only step ready before its tokens are known: ``positions`` names each
        request and the position of its next token (pages reserved). Returns a handle for
        ``step_prepared``, or None when the step cannot simply replay a captured graph (then
        ``step`` runs it as usual). Everything but the tokens is written to the pinned buffer."""
        n = len(positions)
        if not (self.use_graphs and 0 < n <= GRAPH_BATCH_SIZES[-1]):
            return None
        size = next(b for b in GRAPH_BATCH_SIZES if b >= n)
        longest = max(start + 1 for _, start in positions)
        if longest > self._table_width * self.manager.block_size:
            return None
        key = (size, GRAPH_KEY_BUCKET * -(-longest // GRAPH_KEY_BUCKET))
        state = self._graphs.get(key)
        if not isinstance(state, tuple):
            return None
        entries = [StepEntry(seq_id, start, (0,), (0,)) for seq_id, start in positions]
        state[0].fill(entries, self.manager, upload=False)
        return key, entries

    @torch.no_grad()
    def step_prepared(self, handle, tokens) -> torch.Tensor:
        """Run the step that ``prepare_decode`` got ready, now that its tokens are known; every
        entry's logits are returned, float32 [entries, vocab], a view of the graph's output buffer
        that the next step of this shape overwrites. ``tokens``: a sequence of ids, or
        an int32 device tensor (what the sampling kernels of the step before wrote, possibly
        still being computed: the tokens then never visit the host)."""
        key, entries = handle
        if len(tokens) != len(entries):
            raise ValueError(f"{len(tokens)} tokens for {len(entries)} prepared entries")
        self._graphs[key] = self._graphs.pop(key)  # most recently used last
        batch, graph, out = self._graphs[key]
        if isinstance(tokens, torch.Tensor):
            if tokens.dtype != torch.int32 or tokens.device != self.device or tokens.dim() != 1:
                raise ValueError("tokens on the device must be a 1-d int32 tensor on the engine's GPU")
            batch.upload()
            batch.ctx.token_ids[: len(entries)].copy_(tokens)  # after the upload, in stream order
        else:
            for e, tok in zip(entries, tokens):
                if not 0 <= int(tok) < self.spec.vocab_size:
                    raise ValueError(f"request {e.seq_id}: token id {tok} outside the vocabulary")
            batch.set_tokens(tokens)
            batch.upload()
        graph.replay()
        for e in entries:
            self.manager.release_behind_window(e.seq_id, e.start + 1)
        return out[: len(entries)]

    # ------------------------------------------------------------------ the step
    def _forward(self, ctx):
        """The model's step on a laid-out batch: requests that begin in it start from an empty
        fixed-size state (cleared on the device, by the step's own first positions, so that a
        captured step does it too), then the parts run."""
        ctx.products = self.products
        if self.pools.state:
            self.pools.set_fresh_states(ctx.state_slots, ctx.starts, ctx.num_requests)
        return self.model.forward(ctx, self.caches)

    @torch.no_grad()
    def step(self, entries: Sequence[StepEntry]) -> Optional[torch.Tensor]:
        """Run the entries as one batch; float32 logits [wanted, vocab] in the order of the
        entries and of each entry's ``want`` (None when nothing is wanted). The tensor may be a
        view of a replayed graph's own output buffer: it holds this step's logits until the next
        step runs, so a caller that keeps logits across steps copies them."""
        if not entries:
            return None
        if (self.use_graphs and len(entries) <= GRAPH_BATCH_SIZES[-1]
                and all(len(e.tokens) == 1 for e in entries)):
            logits = self._graph_step(entries)
            if logits is not NotImplemented:
                return logits
        if self.use_graphs and len(entries) == 1 and len(entries[0].tokens) > 1:
            logits = self._portion_graph_step(entries[0])
            if logits is not NotImplemented:
                return logits
        if self.use_graphs and 1 < len(entries) <= GRAPH_BATCH_SIZES[-1] + 1:
            logits = self._mixed_graph_step(entries)
            if logits is not NotImplemented:
                return logits
        ctx = build_context(entries, self.manager, self.device, self.spec.vocab_size)
        ctx.num_compute_units = self.num_compute_units
        logits = self._forward(ctx)
        for e in entries:
            self.manager.release_behind_window(e.seq_id, e.start + len(e.tokens))
        return logits
