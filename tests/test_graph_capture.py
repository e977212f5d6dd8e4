"""The host side of HIP-graph capture: what must hold around a capture whatever the GPU does."""

import contextlib
import gc

import pytest
import torch

from clockwork_amd.engine import model_runner
from clockwork_amd.engine.graph_nodes import NODE_KINDS, only_kernels


@pytest.fixture
def stub_graph(monkeypatch):
    """``torch.cuda.graph`` replaced by a context manager that records whether the cyclic garbage
    collector was on while the capture was open."""
    seen = {}

    @contextlib.contextmanager
    def fake_capture(graph, pool=None):
        seen["gc_on_at_begin"] = gc.isenabled()
        yield
        seen["gc_on_at_end"] = gc.isenabled()

    monkeypatch.setattr(torch.cuda, "graph", fake_capture)
    return seen


def test_the_cyclic_collector_is_off_during_a_capture_and_back_afterwards(stub_graph):
    """A collection in the middle of a capture once found an unreachable runner and destroyed its
    captured graphs: HIP calls that a capturing stream refuses, raised from a destructor, which
    ended the process ("operation not permitted when stream is capturing" out of ~CUDAGraph).
    So the collector must be off for as long as a capture is open."""
    assert gc.isenabled()
    with model_runner.capturing(object(), None):
        assert not gc.isenabled()
        # garbage that only the cyclic collector could free stays where it is meanwhile
        cycle = []
        cycle.append(cycle)
        del cycle
    assert stub_graph == {"gc_on_at_begin": False, "gc_on_at_end": False}
    assert gc.isenabled()


def test_the_collector_comes_back_when_the_captured_step_raises(stub_graph):
    with pytest.raises(KeyError):
        with model_runner.capturing(object(), None):
            raise KeyError("a part failed inside the capture")
    assert gc.isenabled()


def test_a_collector_that_was_off_stays_off(stub_graph):
    gc.disable()
    try:
        with model_runner.capturing(object(), None):
            assert not gc.isenabled()
        assert not gc.isenabled()
    finally:
        gc.enable()


def test_only_graphs_of_kernel_nodes_are_kept():
    assert NODE_KINDS[0] == "kernel" and NODE_KINDS[2] == "memset" and NODE_KINDS[1] == "memcpy"
    assert only_kernels({"kernel": 231})
    assert not only_kernels({"kernel": 231, "memset": 1})
    assert not only_kernels({"kernel": 5, "memcpy": 2})


def test_a_block_hands_on_two_outputs_only_to_a_first_norm_that_takes_them():
    """Whether a block may leave two branch outputs pending is asked of the next block's
    arrangement (``first_norm()``), not of a part's name: an arrangement without the hook gets
    one output, one whose first norm does not take pairs gets one, the final norm is asked last."""
    from clockwork_amd.config.spec import LayerSpec, ModelSpec, RunEntry
    from clockwork_amd.parts.model import DecoderModel
    from clockwork_amd.parts.specs import AttentionSpec, RMSNormSpec, SwiGLUSpec

    norm = RMSNormSpec(16, 1e-6)
    layer = LayerSpec("prenorm", AttentionSpec(16, 1, 1, 16, False, False, 0.25), SwiGLUSpec(16, 32), norm, norm)
    model = DecoderModel(ModelSpec("toy", 10, 16, [layer], [RunEntry(0)] * 4, norm))
    asked = []

    class Norm:
        def __init__(self, accepts):
            self.accepts_pending = accepts

    class Block:
        def __init__(self, first):
            self.first = first
            if first is not None:
                self.first_norm = lambda: first

        def forward(self, resid, delta, ctx, cache):
            asked.append(ctx.next_norm_accepts_pending)
            return delta

    class Ctx:
        num_logit_rows = 0
        sequence_positions = positions = None

    # run order 0, 1, 2, 3: block 1 takes pairs, block 2 has no hook, block 3's norm does not take
    # them, then the final norm, which does
    model.layers = [Block(Norm(True)), Block(Norm(True)), Block(None), Block(Norm(False))]
    model.spec.run = [RunEntry(0), RunEntry(1), RunEntry(2), RunEntry(3)]
    model.embedding = type("E", (), {"forward": lambda self, ctx: None})()
    model.final_norm = Norm(True)
    assert model.forward(Ctx(), [None] * 4) is None
    assert asked == [True, False, False, True]
    # the built-in arrangement names its first norm itself
    from clockwork_amd.registry import build_arrangement, build_part

    block = build_arrangement("prenorm", **{name: build_part(part) for name, part in layer.named_parts().items()})
    assert block.first_norm() is block.mixer_norm and block.first_norm().accepts_pending


def test_the_embedding_part_decides_what_positions_are():
    from clockwork_amd.config.spec import LayerSpec, ModelSpec, RunEntry
    from clockwork_amd.parts.model import DecoderModel
    from clockwork_amd.parts.specs import AttentionSpec, RMSNormSpec, SwiGLUSpec

    norm = RMSNormSpec(16, 1e-6)
    layer = LayerSpec("prenorm", AttentionSpec(16, 1, 1, 16, False, False, 0.25), SwiGLUSpec(16, 32), norm, norm)
    model = DecoderModel(ModelSpec("toy", 10, 16, [layer], [RunEntry(0)], norm))
    seen = []

    class Block:
        def forward(self, resid, delta, ctx, cache):
            seen.append(ctx.positions)

    class Ctx:
        num_logit_rows = 0

    model.layers = [Block()]
    for embedding, want in (
        (type("Plain", (), {"forward": lambda self, ctx: None})(), [0, 1, 2]),
        (type("Offset", (), {"forward": lambda self, ctx: None,
                             "positions": lambda self, ctx: ctx.sequence_positions + 2})(), [2, 3, 4]),
    ):
        ctx = Ctx()
        ctx.sequence_positions = ctx.positions = torch.arange(3)
        model.embedding = embedding
        model.forward(ctx, [None])
        assert seen[-1].tolist() == want and ctx.sequence_positions.tolist() == [0, 1, 2]
