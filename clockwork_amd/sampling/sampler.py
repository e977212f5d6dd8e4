"""Token selection above the step function: greedy, temperature, top-k, top-p.

Options and their order are the reference's (clockwork/engine/model_runner.py:134-164):
temperature 0 is the arg-max; otherwise logits / temperature, top-k, top-p, softmax, one
draw. The random stream is counter based: a request's n-th draw is a function of
(seed, n) alone, where the seed is the request's ``SamplingParams.seed`` or the engine's
model seed, so a request samples the same tokens whatever else is in the batch, and
again after a preemption. The kernels are in csrc/sampling.hip.
"""

from __future__ import annotations

from typing import TYPE_CHECKING
from typing import Sequence as Seq

import numpy as np
import torch

from clockwork_amd import ops

if TYPE_CHECKING:
    from clockwork_amd.engine.sequence import Sequence


class Sampler:
    # pinned buffers the rows' options travel through, used in turn: a step's copy may still be
    # under way when the next step's options are written
    _RING = 4
    # batches whose packed options are kept
    _KEPT = 64

    def __init__(self, device, default_seed: int = 0) -> None:
        self.device = device
        self.default_seed = int(default_seed)
        ops.preload(sampling=True)  # compiled now if it has to be, not at the first token
        self._host: list = []     # (pinned int32 buffer, event of its last copy)
        self._next = 0
        self._fixed: dict = {}    # options of a batch that do not change from step to step

    def sample(self, logits: torch.Tensor, seqs: Seq[Sequence]) -> list[int]:
        """One token per row of ``logits`` (float32 [n, vocab]); row i belongs to ``seqs[i]``."""
        drawn = self.launch(logits, seqs)
        return [] if drawn is None else drawn.tolist()

    def _pinned(self, words: int):
        """A pinned int32 buffer of at least ``words`` that no copy is reading any more."""
        if len(self._host) < self._RING:
            self._host.append([torch.empty(max(words, 7 * 64), dtype=torch.int32, pin_memory=True), None])
        slot = self._host[self._next % len(self._host)]
        self._next += 1
        if slot[1] is not None:
            slot[1].synchronize()
        if slot[0].numel() < words:
            slot[0] = torch.empty(words, dtype=torch.int32, pin_memory=True)
        return slot

    def launch(self, logits: torch.Tensor, seqs: Seq[Sequence], pending: int = 0):
        """Start the kernels of ``sample`` and return the tokens as a device tensor (int32 [n]),
        without waiting for them; None for no sequences. ``pending``: tokens of each sequence
        that are sampled already but not yet appended to it (they count as draws made)."""
        n = len(seqs)
        if n == 0:
            return None
        if logits.shape[0] != n:
            raise ValueError(f"{logits.shape[0]} logits rows for {n} sequences")
        # the options of a batch that comes again step after step are packed once: kept under the
        # requests' ids (the entry holds the sequences themselves, and serves only them: an id that
        # has come to mean another request finds nothing), the least recently used entry goes
        key = tuple(s.seq_id for s in seqs)
        fixed = self._fixed.get(key)
        if fixed is not None and not all(a is b for a, b in zip(fixed[3], seqs)):
            fixed = None
        if fixed is None:
            params = [s.sampling_params for s in seqs]
            if all(p.greedy for p in params):
                fixed = None, False, False, list(seqs)
            else:
                vocab = logits.shape[1]
                top_k = np.array([p.top_k if 0 < p.top_k < vocab else -1 for p in params], dtype=np.int32)
                top_p = np.array([p.top_p for p in params], dtype=np.float32)
                seeds = np.array([p.seed if p.seed is not None else self.default_seed for p in params], dtype=np.int64)
                temperature = np.array([p.temperature for p in params], dtype=np.float32)
                # one buffer: seeds, (draws,) temperature, top_p, top_k; the 8-byte items first
                packed = np.concatenate([seeds.view(np.int32), np.zeros(2 * n, dtype=np.int32),
                                         temperature.view(np.int32), top_p.view(np.int32), top_k])
                fixed = packed, bool((top_k > 0).any()), bool((top_p < 1.0).any()), list(seqs)
            self._fixed.pop(key, None)
            while len(self._fixed) >= self._KEPT:
                self._fixed.pop(next(iter(self._fixed)))
        else:
            self._fixed.pop(key)
        self._fixed[key] = fixed   # the newest entry last
        packed, any_top_k, any_top_p, _ = fixed
        if packed is None:
            return ops.argmax(logits)
        slot = self._pinned(7 * n)
        host = slot[0].numpy()
        host[: 7 * n] = packed
        host[2 * n : 4 * n].view(np.int64)[:] = [len(s.output_token_ids) + pending for s in seqs]
        dev = torch.empty(7 * n, dtype=torch.int32, device=self.device)
        dev.copy_(slot[0][: 7 * n], non_blocking=True)
        slot[1] = torch.cuda.Event()
        slot[1].record()
        return ops.sample(
            logits, dev[4 * n : 5 * n].view(torch.float32), dev[6 * n : 7 * n], dev[5 * n : 6 * n].view(torch.float32),
            dev[0 : 2 * n].view(torch.int64), dev[2 * n : 4 * n].view(torch.int64),
            any_top_k=any_top_k, any_top_p=any_top_p,
        )
