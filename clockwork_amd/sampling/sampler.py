"""Token selection above the step function: greedy, temperature, top-k, top-p.

Options and their order are the reference's (clockwork/engine/model_runner.py:134-164):
temperature 0 is the arg-max; otherwise logits / temperature, top-k, top-p, softmax, one
draw. The random stream is counter based: a request's n-th draw is a function of
(seed, n) alone, where the seed is the request's ``SamplingParams.seed`` or the engine's
model seed, so a request samples the same tokens whatever else is in the batch, and
again after a preemption. The kernels are in csrc/sampling.hip.
"""

from __future__ import annotations

from typing import Sequence as Seq

import torch

from clockwork_amd import ops
from clockwork_amd.engine.sequence import Sequence


class Sampler:
    def __init__(self, device, default_seed: int = 0) -> None:
        self.device = device
        self.default_seed = int(default_seed)
        ops.preload(sampling=True)  # compiled now if it has to be, not at the first token

    def sample(self, logits: torch.Tensor, seqs: Seq[Sequence]) -> list[int]:
        """One token per row of ``logits`` (float32 [n, vocab]); row i belongs to ``seqs[i]``."""
        drawn = self.launch(logits, seqs)
        return [] if drawn is None else drawn.tolist()

    def launch(self, logits: torch.Tensor, seqs: Seq[Sequence], pending: int = 0):
        """Start the kernels of ``sample`` and return the tokens as a device tensor (int32 [n]),
        without waiting for them; None for no sequences. ``pending``: tokens of each sequence
        that are sampled already but not yet appended to it (they count as draws made)."""
        n = len(seqs)
        if n == 0:
            return None
        if logits.shape[0] != n:
            raise ValueError(f"{logits.shape[0]} logits rows for {n} sequences")
        params = [s.sampling_params for s in seqs]
        if all(p.greedy for p in params):
            return ops.argmax(logits)
        vocab = logits.shape[1]
        temperature = torch.tensor([p.temperature for p in params], dtype=torch.float32)
        top_k = torch.tensor([p.top_k if 0 < p.top_k < vocab else -1 for p in params], dtype=torch.int32)
        top_p = torch.tensor([p.top_p for p in params], dtype=torch.float32)
        seeds = torch.tensor(
            [p.seed if p.seed is not None else self.default_seed for p in params], dtype=torch.int64
        )
        draws = torch.tensor([len(s.output_token_ids) + pending for s in seqs], dtype=torch.int64)
        dev = self.device
        return ops.sample(
            logits, temperature.to(dev), top_k.to(dev), top_p.to(dev), seeds.to(dev), draws.to(dev),
            any_top_k=bool((top_k > 0).any()), any_top_p=bool((top_p < 1.0).any()),
        )
