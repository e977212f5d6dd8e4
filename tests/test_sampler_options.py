"""The sampler's host side: which kernels a batch's options ask for, and the packed options of a
batch that comes again step after step."""

import pytest
import torch

from clockwork_amd import ops
from clockwork_amd.sampling import sampler as sampler_module
from clockwork_amd.sampling.params import SamplingParams


class _Seq:
    def __init__(self, seq_id, **params):
        self.seq_id = seq_id
        self.sampling_params = SamplingParams(**params)
        self.output_token_ids = []


@pytest.fixture
def sampler(monkeypatch):
    """A sampler whose kernels are stand-ins that record their calls."""
    calls = []
    monkeypatch.setattr(ops, "preload", lambda *a, **k: None)
    monkeypatch.setattr(ops, "argmax", lambda logits: calls.append(("argmax", logits.shape[0])) or torch.zeros(logits.shape[0], dtype=torch.int32))
    made = sampler_module.Sampler("cpu", default_seed=9)
    made.calls = calls
    return made


def test_packed_options_are_kept_per_batch_and_the_oldest_batch_goes(sampler):
    seqs = [_Seq("a", temperature=0.0), _Seq("b", temperature=0.0)]
    sampler.launch(torch.zeros(2, 5), seqs)
    entry = sampler._fixed[("a", "b")]
    sampler.launch(torch.zeros(2, 5), seqs)
    assert sampler._fixed[("a", "b")] is entry and len(sampler._fixed) == 1
    # the same ids, other requests (an id used again after its request ended): packed anew
    others = [_Seq("a", temperature=0.0), _Seq("b", temperature=0.0)]
    sampler.launch(torch.zeros(2, 5), others)
    assert sampler._fixed[("a", "b")] is not entry and sampler._fixed[("a", "b")][3][0] is others[0]
    for i in range(sampler._KEPT + 10):
        sampler.launch(torch.zeros(1, 5), [_Seq(f"r{i}", temperature=0.0)])
        sampler.launch(torch.zeros(2, 5), others)   # in use all along: never the oldest
    assert len(sampler._fixed) == sampler._KEPT
    assert ("a", "b") in sampler._fixed and ("r0",) not in sampler._fixed and (f"r{sampler._KEPT + 9}",) in sampler._fixed
    assert sampler.launch(torch.zeros(0, 5), []) is None
    with pytest.raises(ValueError, match="logits rows"):
        sampler.launch(torch.zeros(3, 5), others)
