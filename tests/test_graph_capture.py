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
