"""The step function: run a batch of (request, its next tokens) from the cache, return logits.

``ModelRunner`` owns the model, the cache manager and the device pools. ``step`` takes
any mix of prompt portions and single decoded tokens, runs exactly the tokens it is
given as one flat batch and returns float32 logits at the wanted places. It samples
nothing: sampling sits above (``clockwork_amd.sampling``), so a replay tool can call
the step raw. The reference's runner ran one forward per prompt and one for all decode
tokens (clockwork/engine/model_runner.py:48-132); here they are one batch.
"""

from __future__ import annotations

from pathlib import Path
from typing import Optional, Sequence

import torch

from clockwork_amd import ops
from clockwork_amd.cache.manager import CacheManager, cache_needs_of, plan_groups
from clockwork_amd.cache.pools import CachePools
from clockwork_amd.config.engine import EngineConfig
from clockwork_amd.engine.batch import StepContext, StepEntry, build_context
from clockwork_amd.parts.model import DecoderModel
from clockwork_amd.registry import resolve_architecture
from clockwork_amd.weights.loader import load_parameters, read_config_json


def require_gpu() -> torch.device:
    if not torch.cuda.is_available():
        raise RuntimeError(
            "clockwork_amd runs on an AMD GPU through its HIP kernels only: no GPU is visible "
            "(torch.cuda.is_available() is False) and there is no CPU path"
        )
    return torch.device("cuda", torch.cuda.current_device())


class ModelRunner:
    def __init__(self, cfg: EngineConfig, weight_source=None, config_dict: Optional[dict] = None,
                 cache_fill: float = 0.0) -> None:
        self.cfg = cfg
        if cfg.model.device not in ("cuda", "cuda:0", "gpu"):
            raise ValueError(f"device {cfg.model.device!r}: this engine runs on the GPU only")
        self.device = require_gpu()
        self.dtype = cfg.model.torch_dtype()
        self.config_dict = config_dict if config_dict is not None else read_config_json(cfg.model.model)
        self.arch = resolve_architecture(self.config_dict)
        self.model_config = self.arch.parse_config(self.config_dict)
        self.spec = self.arch.build_spec(self.model_config)
        self.model = DecoderModel(self.spec)
        ops.preload(self.model.head_dims())
        plan = self.arch.weight_plan(self.model_config, self.spec)
        params = load_parameters(
            cfg.model.model, plan, self.model.param_specs(), self.dtype, self.device, source=weight_source
        )
        self.model.bind(params, self.device, self.dtype)

        groups = plan_groups(cache_needs_of(self.spec, self.model.mixers()))
        self.manager = CacheManager(
            groups,
            block_size=cfg.cache.block_size,
            num_blocks=cfg.cache.num_blocks,
            max_num_seqs=cfg.scheduler.max_num_seqs,
            watermark=cfg.cache.watermark,
        )
        self.pools = CachePools(
            groups, cfg.cache.block_size, cfg.cache.num_blocks, cfg.scheduler.max_num_seqs,
            self.dtype, self.device, fill=cache_fill,
        )
        self.caches = [self.pools.entry_cache(i, e.cache_from) for i, e in enumerate(self.spec.run)]
        self.num_compute_units = torch.cuda.get_device_properties(self.device).multi_processor_count

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

    def release(self, seq_id: str) -> None:
        if self.manager.has(seq_id):
            self.manager.free(seq_id)

    # ------------------------------------------------------------------ the step
    @torch.no_grad()
    def step(self, entries: Sequence[StepEntry]) -> Optional[torch.Tensor]:
        """Run the entries as one batch; float32 logits [wanted, vocab] in the order of the
        entries and of each entry's ``want`` (None when nothing is wanted)."""
        if not entries:
            return None
        if self.manager.state_groups:
            for e in entries:
                if e.start == 0:
                    self.pools.zero_state(self.manager.state_slot(e.seq_id))
        ctx = build_context(entries, self.manager, self.device, self.spec.vocab_size)
        ctx.num_compute_units = self.num_compute_units
        logits = self.model.forward(ctx, self.caches)
        for e in entries:
            self.manager.release_behind_window(e.seq_id, e.start + len(e.tokens))
        return logits
