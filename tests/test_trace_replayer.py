"""The trace replayer's page bookkeeping on the CPU: shares, forks and copies of the trace with
shared pages, run on the real cache manager with a stand-in for the device memory."""

import random

import pytest

from clockwork_amd.cache import CacheManager, plan_groups
from clockwork_amd.config.spec import KVPagesSpec, StateSpec
from clockwork_amd.engine.model_runner import ModelRunner
from clockwork_amd.engine.trace_run import TraceReplayer
from tests import replay


class _Memory:
    """Records what the runner asks of the device pools."""

    def __init__(self):
        self.page_copies, self.state_copies = [], []

    def copy_pages(self, group, pairs):
        self.page_copies += [(group, src, dst) for src, dst in pairs]

    def copy_state(self, src, dst):
        self.state_copies.append((src, dst))


def _runner(needs, block_size, num_blocks):
    runner = ModelRunner.__new__(ModelRunner)  # bookkeeping only: no GPU, no model
    runner.manager = CacheManager(plan_groups(needs), block_size, num_blocks, max_num_seqs=8)
    runner.pools = _Memory()
    runner.steps = []
    runner.step = lambda entries: runner.steps.append(entries)
    return runner


@pytest.mark.parametrize("block_size", [8, 16])
def test_the_shared_trace_copies_pages_and_gives_every_page_back(block_size):
    vocab = 100
    a = [random.Random(1).randrange(vocab) for _ in range(6 * block_size)]
    steps, seqs, starts = replay.shared(a, vocab, block_size)
    assert set(seqs) == {"A", "B", "C", "D", "E", "F", "G"}
    assert seqs["B"][: 2 * block_size] == a[: 2 * block_size] and seqs["D"][: block_size + 3] == a[: block_size + 3]
    runner = _runner([KVPagesSpec(2, 16)] * 2, block_size, 64)
    replayer = TraceReplayer(runner)
    assert starts == {"A": 0, "C": 2 * block_size + block_size // 2 + 1, "B": 2 * block_size, "D": block_size + 3,
                      "G": starts["G"], "E": 0, "F": 0} and starts["G"] > starts["C"]
    seen = {}
    for step in steps:
        live_before = set(replayer.lengths)
        entries, _ = replayer.run_step(step)
        assert len(live_before | {e.seq_id for e in entries}) <= 4 + len(step["end"])
        for e in entries:  # every request's tokens arrive in order, from the shared length on
            assert list(e.tokens) == seqs[e.seq_id][e.start : e.start + len(e.tokens)]
            seen[e.seq_id] = e.start + len(e.tokens)
        runner.manager.audit()
    assert seen == {rid: len(toks) for rid, toks in seqs.items()}
    copies = runner.pools.page_copies
    # A's copy at C's fork, D's out of the page four requests hold, G's at its own fork
    assert len(copies) >= 3 and all(src != dst for _, src, dst in copies)
    assert not runner.manager.live_requests() and runner.manager.min_free_blocks() == 64
    # with exactly the pages of its busiest step the trace still runs, on pages used again
    tight = _runner([KVPagesSpec(2, 16)] * 2, block_size, replayer.peak_pages)
    again = TraceReplayer(tight)
    for step in steps:
        again.run_step(step)
    assert again.peak_pages == replayer.peak_pages and tight.manager.min_free_blocks() == replayer.peak_pages
    assert len(tight.pools.page_copies) == len(copies)


def test_a_share_that_ends_inside_a_page_copies_it_for_the_first_writer():
    runner = _runner([KVPagesSpec(1, 16)], 4, 8)
    replayer = TraceReplayer(runner)
    replayer.run_step({"entries": [{"id": "a", "tokens": list(range(10))}]})
    replayer.run_step({"share": [{"id": "b", "from": "a", "tokens": 6}], "entries": [{"id": "b", "tokens": [7]}]})
    assert runner.manager.block_table("b")[0] == runner.manager.block_table("a")[0]
    assert runner.pools.page_copies == [(0, 1, 3)]  # b wrote position 6 into a copy of a's second page
    replayer.run_step({"entries": [{"id": "a", "tokens": [1]}]})  # a is its page's only holder again
    assert len(runner.pools.page_copies) == 1
    with pytest.raises(ValueError, match="cannot be shared"):
        replayer.run_step({"share": [{"id": "c", "from": "a", "tokens": 12}]})
    with pytest.raises(ValueError, match="live already"):
        replayer.run_step({"fork": [{"id": "b", "from": "a"}]})
    with pytest.raises(ValueError, match="not live"):
        replayer.run_step({"fork": [{"id": "d", "from": "nobody"}]})
    replayer.run_step({"end": ["a", "b"]})
    assert runner.manager.min_free_blocks() == 8


def test_a_fork_copies_fixed_size_state_and_a_share_is_refused_for_such_a_model():
    runner = _runner([KVPagesSpec(1, 16), StateSpec((4,))], 4, 8)
    replayer = TraceReplayer(runner)
    replayer.run_step({"entries": [{"id": "a", "tokens": [1, 2, 3]}]})
    replayer.run_step({"fork": [{"id": "b", "from": "a"}], "entries": [{"id": "b", "tokens": [9]}]})
    assert runner.pools.state_copies == [(runner.manager.state_slot("a"), runner.manager.state_slot("b"))]
    assert runner.pools.page_copies == [(0, 0, 1)]
    with pytest.raises(ValueError, match="cannot share prefixes"):
        replayer.run_step({"share": [{"id": "c", "from": "a", "tokens": 2}]})
    assert not runner.manager.has("c")


def test_random_traces_are_what_they_say():
    """The traces that the GPU tests draw at random: every entry continues its request where the
    last one stopped, at most four requests are live, a fork or a share names a live request that
    holds the tokens it takes, and every request is run to its end and given back."""
    from tests import replay

    kinds = {"share": 0, "fork": 0, "mixed": 0}
    for seed in range(200):
        steps, seqs = replay.random_trace(seed, 512)
        lengths = {}
        for step in steps:
            for share in step["share"]:
                assert 0 < share["tokens"] <= lengths[share["from"]]
                lengths[share["id"]] = share["tokens"]
                kinds["share"] += 1
            for fork in step["fork"]:
                lengths[fork["id"]] = lengths[fork["from"]]
                kinds["fork"] += 1
            for e in step["entries"]:
                at = lengths.get(e["id"], 0)
                assert e["tokens"] and e["tokens"] == seqs[e["id"]][at : at + len(e["tokens"])]
                assert all(0 <= w < len(e["tokens"]) for w in e["want"])
                lengths[e["id"]] = at + len(e["tokens"])
            assert len(lengths) <= 4
            kinds["mixed"] += len(step["entries"]) > 1 and any(len(e["tokens"]) > 1 for e in step["entries"])
            for rid in step["end"]:
                assert lengths.pop(rid) == len(seqs[rid])
        assert not lengths
    assert min(kinds.values()) > 50


def test_the_program_sizes_its_pool_for_max_tokens_in_pages_of_the_given_size():
    from clockwork_amd.engine.trace_run import PAGE, replay_config

    cfg = replay_config("m", "float32", 256)
    assert (cfg.cache.block_size, cfg.cache.num_blocks) == (PAGE, 256 // PAGE) and PAGE == 16
    assert cfg.model.max_model_len == cfg.scheduler.max_model_len == 256   # one request may hold every page
    assert not cfg.cache.enable_prefix_cache and cfg.cache.watermark == 0.0
    cfg = replay_config("m", "bfloat16", 250, page=24)
    assert (cfg.cache.block_size, cfg.cache.num_blocks, cfg.model.max_model_len) == (24, 11, 264)
    assert replay_config("m", "float32", 0, page=8).cache.num_blocks == 1
