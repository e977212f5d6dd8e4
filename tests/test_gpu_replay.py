"""The engine's step function, cache and kernels against the plain implementation: the same
requests whole, with the last 32 tokens decoded one by one, in portions of changing size, and
mixed with other requests on so few pages that pages are used again; float32 and bfloat16."""

import json
import subprocess
import sys
from pathlib import Path

import numpy as np
import pytest
import torch

from tests import replay
from tests.configs import ODD_CONFIGS, TINY_CONFIGS
from tests.plain.qwen2_plain import PlainQwen2

pytestmark = pytest.mark.gpu
REPO = Path(__file__).resolve().parents[1]

# float32 must agree to 1e-5 (the reference's own bar, tests/test_hf_equivalence.py:15-16).
# bfloat16 rounds every activation to 8 bits, which gives each logit an error of about a hundredth
# of the logits' own scale, whatever that scale is (0.15 for the tiny models, above 1 for wide
# ones): its bound is relative to that scale (replay.compare_to_scale: root mean square of the
# errors within 2% of it, the largest within 10%).
TOL = {"float32": dict(rtol=1e-5, atol=1e-5)}


def _check(got, ref, dtype) -> float:
    """Every produced row against the plain implementation; the largest absolute error."""
    if dtype == "float32":
        return replay.compare(got, ref, **TOL["float32"])
    return replay.compare_to_scale(got, ref)[2]

LENGTHS = {"A": [5, 17, 33, 100, 64, 131, 47], "B": [1, 9, 40, 64, 100, 150, 77], "C": [3, 70, 129, 16, 48]}


def _requests(name):
    cfg = TINY_CONFIGS[name][0]
    gen = torch.Generator().manual_seed(len(name) + cfg["vocab_size"])
    return {
        f"r{i}": torch.randint(0, cfg["vocab_size"], (n,), generator=gen).tolist()
        for i, n in enumerate(LENGTHS[name])
    }


_plain_cache = {}


def _plain(name, model_dirs):
    if name not in _plain_cache:
        model = PlainQwen2(model_dirs[name])
        _plain_cache[name] = {rid: model.logits(toks) for rid, toks in _requests(name).items()}
    return _plain_cache[name]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
@pytest.mark.parametrize("mode", ["whole", "prefill_then_decode", "portions", "mixed"])
def test_replay_matches_plain(model_dirs, name, dtype, mode):
    requests = _requests(name)
    block_size = TINY_CONFIGS[name][2]
    live = 4 if mode == "mixed" else 1
    runner = replay.make_runner(model_dirs[name], dtype, block_size, replay.pages_needed(requests, live, block_size))
    steps = getattr(replay, mode)(requests)
    got = replay.run_trace(runner, steps)
    assert len(got) == sum(len(t) for t in requests.values())
    worst = _check(got, _plain(name, model_dirs), dtype)
    print(f"{name} {dtype} {mode}: largest error {worst:.3e}")
    assert not runner.manager.live_requests()
    assert runner.manager.min_free_blocks() == runner.manager.num_blocks


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "A_peaked", "B_peaked"])
def test_requests_that_share_pages_match_plain(model_dirs, name, dtype):
    """Pages held by several requests at once, through the step function: a prefix-cache hit (a
    second request begins with another's first pages while that one is live), a share that ends
    inside a page, two forks in the middle of a page (once the parent writes first and gets the
    copy, once the child), the first owner decoding on after each copy, and strangers that take
    the pages given back, among them copied-from and copied-to ones. Every logit of every
    request against the plain implementation; the pool is NaN-poisoned and, in the second pass,
    holds exactly the pages of the busiest step, so that every given-back page is used again.
    (clockwork/kvcache/block_manager.py:56-83; tests/test_block_manager.py:142-170)"""
    base = name[0]
    cfg, _, block_size = TINY_CONFIGS[base]
    a = torch.randint(0, cfg["vocab_size"], (6 * block_size + 5,), generator=torch.Generator().manual_seed(3)).tolist()
    steps, seqs, _ = replay.shared(a, cfg["vocab_size"], block_size, seed=4)
    plain = PlainQwen2(model_dirs[name])
    ref = {rid: plain.logits(toks) for rid, toks in seqs.items()}
    computed = sum(len(e["tokens"]) for s in steps for e in s["entries"])
    pages = 64
    for attempt in ("roomy", "tight"):
        runner = replay.make_runner(model_dirs[name], dtype, block_size, pages)
        copied = []
        real = runner.pools.copy_pages
        runner.pools.copy_pages = lambda group, pairs: (copied.extend(pairs), real(group, pairs))[1]
        usage = {}
        got = replay.run_trace(runner, steps, usage)
        assert len(got) == computed and len(copied) >= 3
        worst = _check(got, ref, dtype)
        print(f"{name} {dtype} shared pages ({attempt}, {pages} pages, {len(copied)} copies): largest error {worst:.3e}")
        assert not runner.manager.live_requests()
        assert runner.manager.min_free_blocks() == runner.manager.num_blocks
        pages = usage["peak_pages"]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_page_copy_that_misses_one_plane_is_caught(model_dirs, dtype):
    """The negative control of the test above: the copy of a shared page leaves out the values
    of the last layer (one plane of the pool). The comparison must fail."""
    from clockwork_amd import ops

    name = "B_peaked"
    cfg, _, block_size = TINY_CONFIGS["B"]
    a = torch.randint(0, cfg["vocab_size"], (6 * block_size + 5,), generator=torch.Generator().manual_seed(3)).tolist()
    steps, seqs, _ = replay.shared(a, cfg["vocab_size"], block_size, seed=4)
    plain = PlainQwen2(model_dirs[name])
    ref = {rid: plain.logits(toks) for rid, toks in seqs.items()}
    runner = replay.make_runner(model_dirs[name], dtype, block_size, 64, poison=0.0)

    def all_but_the_last_plane(group, pairs):
        pool = runner.pools.kv[group]
        planes = pool.view(pool.shape[0] * 2, pool.shape[2], -1)[:-1]
        ops.copy_pages(planes, torch.tensor(pairs, dtype=torch.int32, device=pool.device))

    runner.pools.copy_pages = all_but_the_last_plane
    got = replay.run_trace(runner, steps)
    with pytest.raises(AssertionError):
        _check(got, ref, dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A_peaked", "B_peaked"])
@pytest.mark.parametrize("mode", ["prefill_then_decode", "portions", "mixed"])
def test_replay_with_peaked_attention(model_dirs, name, dtype, mode):
    """The tiny models with query and key projections scaled up, so that a few keys carry each
    softmax: a key that is missed at a page's edge, read from a stale page or masked wrongly
    moves these logits by their own scale, in bfloat16 too."""
    base = name[0]
    requests = _requests(base)
    block_size = TINY_CONFIGS[base][2]
    live = 4 if mode == "mixed" else 1
    runner = replay.make_runner(model_dirs[name], dtype, block_size, replay.pages_needed(requests, live, block_size))
    got = replay.run_trace(runner, getattr(replay, mode)(requests))
    if name not in _plain_cache:
        model = PlainQwen2(model_dirs[name])
        _plain_cache[name] = {rid: model.logits(toks) for rid, toks in requests.items()}
    worst = _check(got, _plain_cache[name], dtype)
    print(f"{name} {dtype} {mode}: largest error {worst:.3e}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("layers", ["first", "all"])
def test_one_stale_key_at_a_page_edge_is_caught(model_dirs, dtype, layers):
    """The negative control of the peaked models: after a prompt has run, the key of its last
    position in a page is wiped in the cache (in the first layer only, or in all), as if a kernel
    had skipped that slot or read a page that was not the request's. The tokens decoded
    afterwards must fail the comparison that the correct cache passes."""
    name = "B_peaked"
    cfg, _, block_size = TINY_CONFIGS["B"]
    toks = torch.randint(0, cfg["vocab_size"], (120,), generator=torch.Generator().manual_seed(12)).tolist()
    ref = {"x": PlainQwen2(model_dirs[name]).logits(toks)}
    steps = replay.prefill_then_decode({"x": toks}, tail=40)
    for wipe in (False, True):
        runner = replay.make_runner(model_dirs[name], dtype, block_size, 16)
        real = runner.step
        state = {"steps": 0}

        def step(entries):
            out = real(entries)
            state["steps"] += 1
            if wipe and state["steps"] == 1:
                position = 5 * block_size - 1
                page = runner.manager.block_table("x")[position // block_size]
                keys = runner.pools.kv[0][:, 0, page, position % block_size]  # [entries, kv heads, head size]
                (keys[:1] if layers == "first" else keys).zero_()
            return out

        runner.step = step
        got = replay.run_trace(runner, [dict(s) for s in steps])
        if not wipe:
            _check(got, ref, dtype)
        else:
            with pytest.raises(AssertionError):
                _check(got, ref, dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(ODD_CONFIGS))
def test_odd_sizes_replay_like_the_plain_implementation(tmp_path, name, dtype):
    """Head counts, groups, widths and page sizes that the three tiny models do not have."""
    from clockwork_amd.weights.random_init import write_random_model

    cfg, seed, block_size = ODD_CONFIGS[name]
    model_dir = write_random_model(tmp_path / name, cfg, seed)
    gen = torch.Generator().manual_seed(seed)
    requests = {f"r{i}": torch.randint(0, cfg["vocab_size"], (n,), generator=gen).tolist()
                for i, n in enumerate([65, 3, 130, 1, 200, 33])}
    plain = PlainQwen2(model_dir)
    ref = {rid: plain.logits(toks) for rid, toks in requests.items()}
    for mode in ("prefill_then_decode", "mixed"):
        live = 4 if mode == "mixed" else 1
        runner = replay.make_runner(model_dir, dtype, block_size, replay.pages_needed(requests, live, block_size))
        got = replay.run_trace(runner, getattr(replay, mode)(requests))
        assert len(got) == sum(len(t) for t in requests.values())
        worst = _check(got, ref, dtype)
        print(f"{name} {dtype} {mode}: largest error {worst:.3e}")
        assert not runner.manager.live_requests()
        assert runner.manager.min_free_blocks() == runner.manager.num_blocks


@pytest.mark.parametrize("name", ["A", "B"])
@pytest.mark.parametrize("mode", ["prefill_then_decode", "mixed"])
def test_float32_weights_with_full_mantissas(tmp_path, name, mode):
    """The other tests' checkpoints are bfloat16, so their "float32" weights have 8-bit mantissas
    and every product of two of them is exact in float32. Here the folder holds float32 tensors as
    drawn: a float32 path that dropped low bits of its operands anywhere would miss the 1e-5 bar."""
    from clockwork_amd.weights.random_init import write_random_model

    cfg, seed, block_size = TINY_CONFIGS[name]
    model_dir = write_random_model(tmp_path / name, cfg, seed, dtype="float32")
    from safetensors.torch import load_file

    stored = load_file(str(model_dir / "model.safetensors"))
    assert all(t.dtype == torch.float32 for t in stored.values())
    some = stored["model.layers.0.mlp.down_proj.weight"]
    assert float((some.to(torch.bfloat16).float() != some).float().mean()) > 0.9
    requests = _requests(name)
    plain = PlainQwen2(model_dir)
    ref = {rid: plain.logits(toks) for rid, toks in requests.items()}
    live = 4 if mode == "mixed" else 1
    runner = replay.make_runner(model_dir, "float32", block_size, replay.pages_needed(requests, live, block_size))
    assert all(p.dtype == torch.float32 for p in runner.model.params.values())
    got = replay.run_trace(runner, getattr(replay, mode)(requests))
    worst = _check(got, ref, "float32")
    print(f"{name} float32 weights {mode}: largest error {worst:.3e}")


def test_wide_layers_in_float32(tmp_path):
    """The same wide model in true float32, mixed batches: the 1e-5 bar at layer sizes that the
    tiny models do not reach (a feed-forward 4360 wide, 1024-element rows, head size 128)."""
    from clockwork_amd.weights.random_init import write_random_model
    from tests.configs import WIDE

    model_dir = write_random_model(tmp_path / "wide", WIDE, 3)
    gen = torch.Generator().manual_seed(11)
    requests = {f"w{i}": torch.randint(0, WIDE["vocab_size"], (n,), generator=gen).tolist() for i, n in enumerate([40, 70, 55])}
    plain = PlainQwen2(model_dir)
    want = {rid: plain.logits(toks) for rid, toks in requests.items()}
    runner = replay.make_runner(model_dir, "float32", 16, replay.pages_needed(requests, 3, 16))
    got = replay.run_trace(runner, replay.mixed(requests))
    worst = replay.compare(got, want, **TOL["float32"])
    print(f"wide float32 mixed: largest error {worst:.3e}")


@pytest.mark.parametrize("mode", ["prefill_then_decode", "mixed"])
def test_wide_layers_take_the_streaming_and_fused_paths(tmp_path, mode):
    """A model with layers as wide as real ones, so that decode steps run the kernels that tiny
    layers never reach: the persistent streaming product and the second norm fused into the
    gate/up product (eager and as replayed HIP graphs), against the plain implementation."""
    from clockwork_amd import ops
    from clockwork_amd.weights.random_init import write_random_model
    from tests.configs import WIDE

    model_dir = write_random_model(tmp_path / "wide", WIDE, 3)
    lib = ops._load("gemm")
    assert lib.cw_gemm_bf16_swiglu_normed_ok(4, 2 * WIDE["intermediate_size"], WIDE["hidden_size"]) == 1
    calls = {"fused": 0}
    real = lib.cw_gemm_bf16_swiglu_normed

    def counting(*args):
        calls["fused"] += 1
        return real(*args)

    gen = torch.Generator().manual_seed(11)
    requests = {f"w{i}": torch.randint(0, WIDE["vocab_size"], (n,), generator=gen).tolist() for i, n in enumerate([40, 70, 55])}
    plain = PlainQwen2(model_dir)
    want = {rid: plain.logits(toks) for rid, toks in requests.items()}
    live = 3 if mode == "mixed" else 1
    runner = replay.make_runner(model_dir, "bfloat16", 16, replay.pages_needed(requests, live, 16))
    lib.cw_gemm_bf16_swiglu_normed = counting
    try:
        got = replay.run_trace(runner, getattr(replay, mode)(requests))
    finally:
        lib.cw_gemm_bf16_swiglu_normed = real
    assert calls["fused"] > 0
    worst = _check(got, want, "bfloat16")
    print(f"wide bfloat16 {mode}: largest error {worst:.3e}, fused norm launches {calls['fused']}")
    assert not runner.manager.live_requests()


MODES = ["whole", "prefill_then_decode", "portions", "mixed"]


def _benchmark_shape(tmp_path_factory, layers: int):
    """A folder with ``layers`` layers of exactly the benchmark's model (random weights, the full
    vocabulary of 151,936, the tied head), three requests and their logits from the plain
    implementation in float64. Sums of 1,536 and 8,960 float32 products carry rounding of about
    1e-5 themselves, in the engine and in a float32 plain implementation alike (two such
    implementations differ by up to 1.3e-5 after one layer), so the plain side runs in float64:
    what is measured is the engine's own rounding."""
    from clockwork_amd.weights.random_init import write_random_model
    from tests.configs import LAYER_1P5B

    config = dict(LAYER_1P5B, num_hidden_layers=layers)
    model_dir = write_random_model(tmp_path_factory.mktemp(f"benchmark_shape_{layers}") / "model", config, 2)
    gen = torch.Generator().manual_seed(11)
    requests = {f"w{i}": torch.randint(0, config["vocab_size"], (n,), generator=gen).tolist()
                for i, n in enumerate([40, 70, 55])}
    plain = PlainQwen2(model_dir, dtype=torch.float64)
    want = {rid: plain.logits(toks).float() for rid, toks in requests.items()}
    return model_dir, requests, want


@pytest.fixture(scope="module")
def benchmark_layer(tmp_path_factory):
    return _benchmark_shape(tmp_path_factory, 1)


@pytest.fixture(scope="module")
def benchmark_model(tmp_path_factory):
    return _benchmark_shape(tmp_path_factory, 28)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("mode", MODES)
def test_a_layer_of_the_benchmark_model(benchmark_layer, mode, dtype):
    """One layer with exactly the sizes of the benchmark's model, in every way of cutting the
    work: float32 at the 1e-5 bar (25 million logits), bfloat16 within its bound."""
    model_dir, requests, want = benchmark_layer
    live = 3 if mode == "mixed" else 1
    runner = replay.make_runner(model_dir, dtype, 16, replay.pages_needed(requests, live, 16))
    got = replay.run_trace(runner, getattr(replay, mode)(requests))
    assert len(got) == 165
    worst = _check(got, want, dtype)
    print(f"benchmark layer {dtype} {mode}: largest error {worst:.3e}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("mode", MODES)
def test_the_whole_benchmark_model(benchmark_model, mode, dtype):
    """All 28 layers of the benchmark's model (a 3 GB folder, 1.5 billion random parameters), in
    every way of cutting the work, against the plain implementation in float64 on the CPU.
    float32: the 1e-5 bar and the same arg-max at every position. bfloat16: the rounding of 28
    layers adds up to about 2% of the logits' scale (root mean square; bound 4%, the largest of 25
    million within 20%: 12 to 18% were measured over the four ways), and wherever the arg-max differs the plain logits of the two tokens lie
    closer than a tenth of the scale (random weights give many near-ties)."""
    model_dir, requests, want = benchmark_model
    live = 3 if mode == "mixed" else 1
    runner = replay.make_runner(model_dir, dtype, 16, replay.pages_needed(requests, live, 16))
    got = replay.run_trace(runner, getattr(replay, mode)(requests))
    del runner
    assert len(got) == 165
    gaps = []
    for (rid, pos), row in got.items():
        ref = want[rid][pos]
        a, b = int(row.argmax()), int(ref.argmax())
        if a != b:
            gaps.append(float(ref[b] - ref[a]))
    if dtype == "float32":
        worst = replay.compare(got, want, **TOL["float32"])
        assert not gaps
        print(f"whole model float32 {mode}: largest error {worst:.3e}")
    else:
        scale, rms, worst = replay.compare_to_scale(got, want, rms_bound=4e-2, worst_bound=2e-1)
        print(f"whole model bfloat16 {mode}: scale {scale:.3f}, rms {rms:.3e}, largest {worst:.3e}, arg-max differs at {len(gaps)} of 165")
        assert all(g < 1e-1 * scale for g in gaps) and len(gaps) < 30


# ------------------------------------------------------------------ the steps the benchmark times
@pytest.fixture(scope="module")
def benchmark_steps(tmp_path_factory):
    """One layer of the benchmark model's widths with a small vocabulary and peaked attention (a
    key that is missed or read twice moves the logits by their own scale), and the requests of
    the benchmark's two kinds of decode step: eight that hold 2048-token prompts, sixty-four that
    hold about 600 tokens (sixteen different sequences, four requests each). Plain logits in
    float64 at the positions that are decoded."""
    from clockwork_amd.weights.random_init import write_random_model
    from tests.configs import LAYER_1P5B

    config = dict(LAYER_1P5B, vocab_size=1203)
    root = tmp_path_factory.mktemp("benchmark_steps")
    model_dir = replay.sharpen(write_random_model(root / "base", config, 2), root / "peaked")
    gen = torch.Generator().manual_seed(31)
    draw = lambda n: torch.randint(0, config["vocab_size"], (n,), generator=gen).tolist()
    eight = {f"e{i}": draw(2048 + 12) for i in range(8)}
    distinct = [draw(590 + i) for i in range(16)]
    many = {f"m{i}": distinct[i % 16] for i in range(64)}
    plain = PlainQwen2(model_dir, dtype=torch.float64)
    want = {}
    for rid, toks in eight.items():
        want[rid] = {2047 + j: row for j, row in enumerate(plain.logits(toks)[2047:].float())}
    rows = [plain.logits(toks)[len(toks) - 5 :].float() for toks in distinct]
    for i, (rid, toks) in enumerate(many.items()):
        want[rid] = {len(toks) - 5 + j: row for j, row in enumerate(rows[i % 16])}
    return model_dir, eight, many, want


def _prompts_then_decode(requests: dict, decoded: int, per_step: int) -> list:
    """The prompts, ``per_step`` requests a step and each whole, then the last ``decoded`` tokens
    of all requests side by side, one a step; the logits of every decoded position and of the
    prompts' last tokens are wanted."""
    ids = list(requests)
    steps = []
    for at in range(0, len(ids), per_step):
        steps.append({"entries": [{"id": r, "tokens": requests[r][: len(requests[r]) - decoded],
                                   "want": [len(requests[r]) - decoded - 1]} for r in ids[at : at + per_step]], "end": []})
    for j in range(decoded, 0, -1):
        steps.append({"entries": [{"id": r, "tokens": [requests[r][len(requests[r]) - j]], "want": [0]} for r in ids], "end": []})
    steps[-1]["end"] = ids
    return steps


def _watch_attention(monkeypatch):
    """Record how the attention kernels for single tokens are asked to cut the keys."""
    from clockwork_amd import ops

    calls = {"decode": [], "tile": []}
    real_decode, real_tile = ops.attention_decode, ops.attention

    def decode(**kw):
        calls["decode"].append((kw["n_items"], kw["n_splits"], kw["split_keys"], kw["identity"]))
        return real_decode(**kw)

    def tile(**kw):
        if kw["rows"] == 16:
            calls["tile"].append((kw["n_items"], kw["n_splits"]))
        return real_tile(**kw)

    monkeypatch.setattr(ops, "attention_decode", decode)
    monkeypatch.setattr(ops, "attention", tile)
    return calls


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decode_steps_of_eight_behind_2048_token_prompts(benchmark_steps, monkeypatch, dtype):
    """What the benchmark's headline number times, at its widths: 2048-token prompts as portions
    of the whole token budget (the third and later ones replay a captured graph), then decode steps
    of all eight requests (the first eager, the second captured, ten replayed), each request's
    keys cut into sixteen splits at fixed places and merged; NaN-poisoned pools; every decoded
    position against the plain implementation."""
    model_dir, eight, _, want = benchmark_steps
    calls = _watch_attention(monkeypatch)
    runner = replay.make_runner(model_dir, dtype, 16, replay.pages_needed(eight, 8, 16), max_model_len=4096)
    got = replay.run_trace(runner, _prompts_then_decode(eight, 12, 1))
    assert len(got) == 8 * 13
    worst = _check(got, want, dtype)
    captured = [k for k, v in runner._graphs.items() if isinstance(v, tuple)]
    assert (8, 2560) in captured and any(k[0] == "portion" and k[1] == 2048 for k in captured), captured
    if dtype == "bfloat16":
        cuts = [c for c in calls["decode"] if c[0] == 8]
        # sixteen splits (16 workgroups a split: one for every compute unit): of 160 keys in the
        # eager step, which plans for its 2049 keys, and in the graph, planned for its 2560-key bucket
        assert cuts and all(n_splits == 16 and split_keys == 160 and identity for _, n_splits, split_keys, identity in cuts), cuts
        assert len(cuts) >= 2  # the eager step and the capture
    else:
        cuts = [c for c in calls["tile"] if c[0] == 8]
        assert cuts and all(n_splits > 1 for _, n_splits in cuts), cuts
    print(f"decode of eight behind 2048 tokens, {dtype}: largest error {worst:.3e}, cuts {cuts[0]}")
    assert not runner.manager.live_requests()


def test_key_ranges_that_miss_keys_are_caught(benchmark_steps, monkeypatch):
    """The negative control of the test above: every split's range of keys is 32 keys shorter
    than planned and begins that much earlier for every split before it, so the last 512 keys
    of a context are read by nobody. The comparison must fail."""
    from clockwork_amd import ops

    model_dir, eight, _, want = benchmark_steps
    real = ops.attention_decode

    def shifted(**kw):
        if kw["split_keys"] > 32:
            kw["split_keys"] -= 32
            kw["max_ctx"] = kw["n_splits"] * kw["split_keys"]
        return real(**kw)

    monkeypatch.setattr(ops, "attention_decode", shifted)
    runner = replay.make_runner(model_dir, "bfloat16", 16, replay.pages_needed(eight, 8, 16), max_model_len=4096, use_graphs=False)
    got = replay.run_trace(runner, _prompts_then_decode(eight, 12, 1))
    with pytest.raises(AssertionError):
        _check({k: v for k, v in got.items() if k[1] > 2047}, want, "bfloat16")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decode_steps_of_sixty_four(benchmark_steps, monkeypatch, dtype):
    """The benchmark's wide batch: 64 requests that hold about 600 tokens decode side by side
    (eager, captured, replayed twice), two splits a request in bfloat16."""
    model_dir, _, many, want = benchmark_steps
    calls = _watch_attention(monkeypatch)
    runner = replay.make_runner(model_dir, dtype, 16, replay.pages_needed(many, 64, 16), max_model_len=4096)
    got = replay.run_trace(runner, _prompts_then_decode(many, 4, 3))
    assert len(got) == 64 * 5
    worst = _check(got, want, dtype)
    assert isinstance(runner._graphs.get((64, 1024)), tuple), list(runner._graphs)
    if dtype == "bfloat16":
        cuts = [c for c in calls["decode"] if c[0] == 64]
        assert cuts and all(n_splits > 1 and identity for _, n_splits, _, identity in cuts), cuts
    else:
        cuts = [c for c in calls["tile"] if c[0] == 64]
        assert cuts
    print(f"decode of 64 behind 600 tokens, {dtype}: largest error {worst:.3e}, cuts {cuts[0]}")
    assert not runner.manager.live_requests()


def test_a_long_portion_takes_the_wide_tile_product(tmp_path):
    """A prompt of 1,300 tokens through a layer with the benchmark model's widths, bfloat16: run
    whole, its gate/up product goes through the package's own wide-tile kernel (1,300 rows: 6 row
    tiles, the last one a third full); run in portions of 300 through the library and the gate
    kernel; a second prompt rides beside the long one's last portion. Both against the plain
    implementation, and the two ways against each other."""
    from clockwork_amd import ops
    from clockwork_amd.weights.random_init import write_random_model
    from tests.configs import LAYER_1P5B

    config = dict(LAYER_1P5B, vocab_size=1203, tie_word_embeddings=False)
    model_dir = write_random_model(tmp_path / "model", config, 5)
    gen = torch.Generator().manual_seed(17)
    long = torch.randint(0, 1203, (1300,), generator=gen).tolist()
    short = torch.randint(0, 1203, (1100,), generator=gen).tolist()
    plain = PlainQwen2(model_dir)
    want = {"long": plain.logits(long), "short": plain.logits(short)}
    want["other"] = want["long"][:200]   # the long prompt's first 200 tokens as a request of their own
    wanted = [0, 1, 255, 256, 257, 700, 1023, 1024, 1279, 1280, 1298, 1299]
    calls = []
    real = ops.linear_tiled
    ops.linear_tiled = lambda *a, **k: (calls.append((a[0].shape[0], k.get("wide"))), real(*a, **k))[1]
    try:
        runner = replay.make_runner(model_dir, "bfloat16", 16, 170, max_model_len=2048)
        whole = replay.run_trace(runner, [
            {"entries": [{"id": "long", "tokens": long, "want": wanted}], "end": ["long"]},
            # 1,100 + 200 rows in one step: two requests share the product's row tiles
            {"entries": [{"id": "short", "tokens": short, "want": [w for w in wanted if w < 1100]},
                         {"id": "other", "tokens": long[:200], "want": [0, 199]}], "end": ["short", "other"]},
        ])
        assert calls == [(1300, True), (1300, True)]
        calls.clear()
        steps = [{"entries": [{"id": "long", "tokens": long[at : at + 300], "want": [w - at for w in wanted if at <= w < at + 300]}],
                  "end": []} for at in range(0, 1300, 300)]
        steps[-1]["end"] = ["long"]
        cut = replay.run_trace(runner, steps)
        assert not calls
    finally:
        ops.linear_tiled = real
    assert len(whole) == len(wanted) + sum(w < 1100 for w in wanted) + 2 and len(cut) == len(wanted)
    # 450 tokens as a step of their own replay the graph for 512 rows, which holds the wide-tile
    # kernel: the first run is eager, the second is captured, the third replays
    for turn in range(3):
        calls.clear()
        ops.linear_tiled = lambda *a, **k: (calls.append((a[0].shape[0], k.get("wide"))), real(*a, **k))[1]
        try:
            again = replay.run_trace(runner, [{"entries": [{"id": "g", "tokens": long[:450], "want": [449]}], "end": ["g"]}])
        finally:
            ops.linear_tiled = real
        # eager with its own 450 rows (the library's product), captured with 512, then replayed
        assert (set(calls) == {(512, True)}) if turn == 1 else not calls, (turn, calls)
        replay.compare_to_scale(again, {"g": want["long"]})
    replay.compare_to_scale(whole, want)
    replay.compare_to_scale(cut, want)
    replay.compare_to_scale(cut, {"long": {p: whole[("long", p)] for p in wanted}})


@pytest.mark.parametrize("which", ["LAYER_7B", "LAYER_32B"])
def test_layers_of_the_larger_models(tmp_path, which):
    """One layer of the 7B and of the 32B shape, bfloat16: a prompt in two portions, then tokens
    one by one beside a second request's prompt, against the plain implementation."""
    from clockwork_amd.weights.random_init import write_random_model
    from tests import configs

    config = getattr(configs, which)
    model_dir = write_random_model(tmp_path / which, config, 7)
    gen = torch.Generator().manual_seed(13)
    requests = {f"m{i}": torch.randint(0, config["vocab_size"], (n,), generator=gen).tolist() for i, n in enumerate([45, 21])}
    plain = PlainQwen2(model_dir)
    want = {rid: plain.logits(toks) for rid, toks in requests.items()}
    a, b = requests["m0"], requests["m1"]
    steps = [
        {"entries": [{"id": "m0", "tokens": a[:30], "want": list(range(30))}], "end": []},
        {"entries": [{"id": "m0", "tokens": a[30:37], "want": list(range(7))}], "end": []},
    ]
    for p in range(37, 45):
        entry = [{"id": "m0", "tokens": a[p : p + 1], "want": [0]}]
        if p == 39:
            entry.append({"id": "m1", "tokens": b[:17], "want": list(range(17))})
        if p > 39 and 17 + (p - 40) < len(b):
            q = 17 + (p - 40)
            entry.append({"id": "m1", "tokens": b[q : q + 1], "want": [0]})
        steps.append({"entries": entry, "end": []})
    steps[-1]["end"] = ["m0", "m1"]
    runner = replay.make_runner(model_dir, "bfloat16", 16, 16)
    got = replay.run_trace(runner, steps)
    assert len(got) == 45 + 17 + 4
    # Rounding every activation to 8 bits gives each logit an error of about a hundredth of the
    # logits' own scale (measured: 0.95% and 1.0% for the two shapes, the same at every position
    # and in every kind of step), and that scale grows with the width (1.2 and 1.4 here, 0.15 for
    # the tiny models, whose bound is absolute). So the bound is relative to the scale: the root
    # mean square of the errors within 2% of it, the largest of the 100,000 within 10%. A wrong
    # key, mask or weight row moves logits by the scale itself.
    scale = torch.cat([w.flatten() for w in want.values()]).square().mean().sqrt().item()
    errors = torch.stack([row - want[rid][pos] for (rid, pos), row in sorted(got.items())])
    assert not torch.isnan(errors).any()
    rms, worst = errors.square().mean().sqrt().item(), errors.abs().max().item()
    print(f"{which} bfloat16: logits' scale {scale:.3f}, rms error {rms:.3e}, largest {worst:.3e}")
    assert rms < 2e-2 * scale and worst < 1e-1 * scale


def test_replay_with_the_tiled_products_instead_of_the_library(model_dirs):
    """``hip_products``: the large bfloat16 products run on the package's own tiled kernel."""
    from clockwork_amd import ops
    from clockwork_amd.config.engine import EngineConfig
    from clockwork_amd.engine.model_runner import ModelRunner

    name = "B"
    requests = _requests(name)
    cfg = EngineConfig.defaults(str(model_dirs[name]), dtype="bfloat16", block_size=8, enable_prefix_cache=False,
                                watermark=0.0, max_model_len=512, hip_products=True,
                                num_blocks=replay.pages_needed(requests, 4, 8))
    calls = []
    real = ops.linear_tiled
    ops.linear_tiled = lambda *a, **k: (calls.append(1), real(*a, **k))[1]
    try:
        runner = ModelRunner(cfg, cache_fill=float("nan"))
        got = replay.run_trace(runner, replay.mixed(requests))
    finally:
        ops.linear_tiled = real
    assert calls and runner.products.hip_products and not ops.DEFAULT_POLICY.hip_products
    _check(got, _plain(name, model_dirs), "bfloat16")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_first_tokens_and_long_decoding(model_dirs, dtype):
    """The first tokens of a sequence (one-token prompt, then decoding from position 1) and a
    long run of single tokens across many page edges."""
    name = "B"
    cfg, _, block_size = TINY_CONFIGS[name]
    toks = torch.randint(0, cfg["vocab_size"], (200,), generator=torch.Generator().manual_seed(7)).tolist()
    runner = replay.make_runner(model_dirs[name], dtype, block_size, -(-200 // block_size))
    steps = [{"entries": [{"id": "x", "tokens": [t], "want": [0]}], "end": []} for t in toks]
    got = replay.run_trace(runner, steps)
    ref = {"x": PlainQwen2(model_dirs[name]).logits(toks)}
    _check(got, ref, dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A_peaked", "B_peaked", "C"])
def test_random_traces_match_plain(model_dirs, name, dtype):
    """Twenty random traces a model (replay.random_trace: portions and single tokens in any mix,
    requests left out of steps, forks and shares cut at any token, logits wanted at random
    places), on page pools that hold the four longest requests and little more, so that pages are
    used again and again. Every wanted row is compared with the plain implementation."""
    cfg, _, block_size = TINY_CONFIGS[name.split("_")[0]]
    model = PlainQwen2(model_dirs[name])
    rows = 0
    for seed in range(20):
        steps, seqs = replay.random_trace(1000 * len(name) + seed, cfg["vocab_size"])
        longest = sorted((-(-len(t) // block_size) for t in seqs.values()), reverse=True)[:4]
        runner = replay.make_runner(model_dirs[name], dtype, block_size, sum(longest) + len(seqs) + 2, max_model_len=1024)
        got = replay.run_trace(runner, steps)
        ref = {rid: model.logits(toks) for rid, toks in seqs.items()}
        _check(got, ref, dtype)
        assert not runner.manager.live_requests()
        assert runner.manager.min_free_blocks() == runner.manager.num_blocks
        rows += len(got)
    assert rows > 500


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["B_peaked", "C"])
def test_short_portions_behind_a_long_prefix(model_dirs, name, dtype):
    """Portions of 2 to 170 tokens behind 700 to 1100 cached ones make few attention workgroups with
    long key ranges: in bfloat16 the plan shares every item's keys among several workgroups and a
    second kernel puts their parts together. Every token's logits are compared, with attention that
    looks at single far keys (B_peaked); a second request decodes beside some of the portions,
    which come twice in the same shape so that they also run as captured graphs."""
    from clockwork_amd.engine.batch import StepContext
    from clockwork_amd.parts.attention import attention_plan

    cfg, _, block_size = TINY_CONFIGS[name.split("_")[0]]
    gen = torch.Generator().manual_seed(46)
    toks = {"x": torch.randint(0, cfg["vocab_size"], (1100,), generator=gen).tolist(),
            "d": torch.randint(0, cfg["vocab_size"], (60,), generator=gen).tolist()}
    steps = [{"entries": [{"id": "x", "tokens": toks["x"][:700], "want": [699]}], "end": []},
             {"entries": [{"id": "d", "tokens": toks["d"][:40], "want": [39]}], "end": []}]
    at, d_at = 700, 40
    for i, n in enumerate([3, 17, 17, 64, 100, 40, 40, 2, 117]):
        entries = [{"id": "x", "tokens": toks["x"][at : at + n], "want": list(range(n))}]
        if i % 2:
            entries.insert(0, {"id": "d", "tokens": toks["d"][d_at : d_at + 1], "want": [0]})
            d_at += 1
        steps.append({"entries": entries, "end": []})
        at += n
    assert at == 1100
    steps[-1]["end"] = ["x", "d"]
    # the plan of such a step cuts its items (heads as in the model, 256 compute units)
    probe = StepContext()
    probe.device = torch.device("cuda")
    probe.h_q_lens, probe.h_ctx_lens = [64], [800]
    assert attention_plan(probe, cfg["num_attention_heads"], cfg["num_key_value_heads"], narrow_ok=True).mfma_parts >= 2
    runner = replay.make_runner(model_dirs[name], dtype, block_size, -(-1100 // block_size) + -(-60 // block_size) + 2,
                                max_model_len=1200)
    got = replay.run_trace(runner, steps)
    model = PlainQwen2(model_dirs[name])
    ref = {k: model.logits(v) for k, v in toks.items()}
    assert len(got) == 2 + 400 + 4
    _check(got, ref, dtype)


@pytest.mark.parametrize("dtype,graph_limit", [("float32", None), ("bfloat16", None), ("bfloat16", 1)])
def test_graph_replays_equal_eager_steps(model_dirs, dtype, graph_limit, monkeypatch):
    """Decode steps replay a captured HIP graph. Every replay is checked against the same step run
    eagerly by a second runner, over many replays with eager work (prompt portions of another
    request, a request ending and its pages going to a new one) and synchronisations in between.
    With room for one graph only, the two batch shapes keep pushing each other out."""
    from clockwork_amd.engine import model_runner

    if graph_limit is not None:
        monkeypatch.setattr(model_runner, "GRAPH_LIMIT", graph_limit)
    name = "B"
    cfg, _, block_size = TINY_CONFIGS[name]
    gen = torch.Generator().manual_seed(21)
    toks = {k: torch.randint(0, cfg["vocab_size"], (n,), generator=gen).tolist() for k, n in
            {"a": 90, "b": 75, "c": 60, "d": 41}.items()}
    steps = [{"entries": [{"id": "a", "tokens": toks["a"][:30], "want": [29]}, {"id": "b", "tokens": toks["b"][:20], "want": [19]}], "end": []}]
    at = {"a": 30, "b": 20, "c": 0, "d": 0}

    def one(ids):
        entries = []
        for i in ids:
            entries.append({"id": i, "tokens": toks[i][at[i] : at[i] + 1], "want": [0]})
            at[i] += 1
        return entries

    for i in range(55):
        if i % 7 == 3 and at["c"] < 40:  # an eager step: a portion of c beside the single tokens
            entries = one(["a", "b"]) + [{"id": "c", "tokens": toks["c"][at["c"] : at["c"] + 10], "want": [9]}]
            at["c"] += 10
            steps.append({"entries": entries, "end": []})
        elif at["b"] == len(toks["b"]) - 1:
            steps.append({"entries": one(["a", "b"]), "end": ["b"]})
        elif at["b"] >= len(toks["b"]):
            ids = ["a", "c"] + (["d"] if i % 2 else [])  # batch sizes 2 and 3: two graph shapes
            steps.append({"entries": one([x for x in ids if at[x] < len(toks[x])]), "end": []})
        else:
            steps.append({"entries": one(["a", "b"]), "end": []})
    pages = 40
    with_graphs = replay.make_runner(model_dirs[name], dtype, block_size, pages, use_graphs=True)
    eager = replay.make_runner(model_dirs[name], dtype, block_size, pages, use_graphs=False)
    got_g = replay.run_trace(with_graphs, [dict(s) for s in steps])
    got_e = replay.run_trace(eager, [dict(s) for s in steps])
    captured = [k for k, v in with_graphs._graphs.items() if isinstance(v, tuple)]
    assert captured, "no graph was captured"
    assert graph_limit is None or len(captured) <= graph_limit
    assert got_g.keys() == got_e.keys() and len(got_g) > 100
    # the graph plans its attention splits for a padded batch and a context bucket, so sums may be
    # taken in another order than in the eager step: equal up to that rounding, far inside the
    # bar that both must meet against the plain implementation
    # (bfloat16: within 3% of the logits' own scale, whatever that scale is)
    scale = torch.stack(list(got_e.values())).square().mean().sqrt().item()
    close = dict(rtol=2e-6, atol=2e-6) if dtype == "float32" else dict(rtol=0.0, atol=3e-2 * scale)
    for key in got_e:
        torch.testing.assert_close(got_g[key], got_e[key], **close, msg=lambda m: f"graph replay differs from the eager step at {key}: {m}")
    model = PlainQwen2(model_dirs[name])
    ref = {k: model.logits(v) for k, v in toks.items()}
    _check(got_g, ref, dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_full_budget_portions_replay_as_graphs(model_dirs, dtype):
    """A step that is one request's portion of exactly the token budget replays a captured graph
    from its third occurrence on. Two long prompts are cut into such portions (the last one of
    each is shorter and runs eagerly), with decode steps, another request's short prompt and a
    request ending in between; logits are wanted for the last token of some portions and for none
    of others (two graph shapes). Every step is checked against a runner without graphs and
    against the plain implementation."""
    from clockwork_amd.config.engine import EngineConfig
    from clockwork_amd.engine.model_runner import ModelRunner

    name = "B"
    cfg, _, block_size = TINY_CONFIGS[name]
    budget = 72  # more rows than the narrow products take, and not a multiple of the page size
    gen = torch.Generator().manual_seed(33)
    toks = {k: torch.randint(0, cfg["vocab_size"], (n,), generator=gen).tolist() for k, n in
            {"a": 6 * budget + 17, "b": 4 * budget + 5, "c": 30}.items()}
    steps = []
    at = {k: 0 for k in toks}

    def portion(rid, n, want_last):
        e = {"id": rid, "tokens": toks[rid][at[rid] : at[rid] + n], "want": [n - 1] if want_last else []}
        at[rid] += n
        return e

    for i in range(6):
        steps.append({"entries": [portion("a", budget, i % 2 == 0)], "end": []})
        if i == 1:
            steps.append({"entries": [portion("c", 29, True)], "end": []})
        if i >= 1 and at["c"] < len(toks["c"]):
            steps.append({"entries": [portion("c", 1, True)], "end": ["c"]})
        if i < 4:
            steps.append({"entries": [portion("b", budget, i % 2 == 1)], "end": []})
    steps.append({"entries": [portion("a", 17, True), portion("b", 5, True)], "end": ["a", "b"]})
    assert all(at[k] == len(v) for k, v in toks.items())

    def runner(use_graphs):
        ecfg = EngineConfig.defaults(
            str(model_dirs[name]), dtype=dtype, block_size=block_size, num_blocks=160, enable_prefix_cache=False,
            watermark=0.0, max_model_len=512, max_num_batched_tokens=budget,
        )
        return ModelRunner(ecfg, cache_fill=float("nan"), use_graphs=use_graphs)

    with_graphs, eager = runner(True), runner(False)
    got_g = replay.run_trace(with_graphs, [dict(s) for s in steps])
    got_e = replay.run_trace(eager, [dict(s) for s in steps])
    captured = [k for k, v in with_graphs._graphs.items() if isinstance(v, tuple) and k[0] == "portion"]
    assert len(captured) == 2, f"portion graphs captured: {captured}"
    assert got_g.keys() == got_e.keys() and len(got_g) >= 8
    for key in got_e:  # the same kernels in the same order: the same numbers
        torch.testing.assert_close(got_g[key], got_e[key], rtol=0, atol=0, msg=lambda m: f"portion graph differs from the eager step at {key}: {m}")
    model = PlainQwen2(model_dirs[name])
    ref = {k: model.logits(v) for k, v in toks.items()}
    _check(got_g, ref, dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_short_prompts_replay_padded_graphs(model_dirs, dtype):
    """A step that is one request's portion of 2 to 512 tokens replays a graph captured for the
    next of a few sizes: the rows past the portion belong to no request. Prompts of many lengths
    around those sizes, each followed by a second portion (so the padded step also runs behind
    cached keys, and its own keys are read back) and a few single tokens; the pools are poisoned
    with NaN, so a read past a request's tokens would show. Checked against a runner without
    graphs and against the plain implementation."""
    from clockwork_amd.config.engine import EngineConfig
    from clockwork_amd.engine.model_runner import ModelRunner

    name = "C"
    cfg, _, block_size = TINY_CONFIGS[name]
    gen = torch.Generator().manual_seed(44)
    firsts = [65, 100, 128, 129, 127, 70, 200, 256, 257, 300, 384, 90, 500, 512, 260, 130, 2, 3, 16, 17, 33, 40, 64, 9, 20, 31]
    toks, steps = {}, []
    for i, n in enumerate(firsts):
        rid = f"r{i}"
        second = 66 + (i * 37) % 120
        toks[rid] = torch.randint(0, cfg["vocab_size"], (n + second + 3,), generator=gen).tolist()
        steps.append({"entries": [{"id": rid, "tokens": toks[rid][:n], "want": [n - 1]}], "end": []})
        steps.append({"entries": [{"id": rid, "tokens": toks[rid][n : n + second], "want": [second - 1] if i % 2 else []}], "end": []})
        for j in range(3):
            at = n + second + j
            steps.append({"entries": [{"id": rid, "tokens": toks[rid][at : at + 1], "want": [0]}], "end": [rid] if j == 2 else []})

    def runner(use_graphs):
        ecfg = EngineConfig.defaults(
            str(model_dirs[name]), dtype=dtype, block_size=block_size, num_blocks=64, enable_prefix_cache=False,
            watermark=0.0, max_model_len=1024,
        )
        return ModelRunner(ecfg, cache_fill=float("nan"), use_graphs=use_graphs)

    with_graphs, eager = runner(True), runner(False)
    got_g = replay.run_trace(with_graphs, [dict(s) for s in steps])
    got_e = replay.run_trace(eager, [dict(s) for s in steps])
    captured = sorted(k[1] for k, v in with_graphs._graphs.items() if isinstance(v, tuple) and k[0] == "portion")
    assert set(captured) >= {16, 32, 64, 128, 256, 384, 512}, f"portion graphs captured: {captured}"
    assert got_g.keys() == got_e.keys()
    # padded steps run products of more rows than the eager ones, so another kernel may take them,
    # and the single tokens' graphs split their keys otherwise than eager steps: equal up to rounding
    close = dict(rtol=2e-6, atol=2e-6) if dtype == "float32" else dict(rtol=2e-2, atol=2e-2)
    for key in got_e:
        torch.testing.assert_close(got_g[key], got_e[key], **close, msg=lambda m: f"padded graph differs from the eager step at {key}: {m}")
    model = PlainQwen2(model_dirs[name])
    ref = {k: model.logits(v) for k, v in toks.items()}
    _check(got_g, ref, dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["B", "C"])
def test_single_tokens_beside_a_portion_replay_padded_graphs(model_dirs, name, dtype):
    """Decoding requests beside one request's portion replay a graph captured for the next batch
    size and the next portion size. Three, then five decoding requests (one joins after every
    prompt, so the batch sizes 4 and 8 are used and left partly empty); prompts arrive one after the
    other with lengths around the portion sizes, each in one step (its last token's logits wanted)
    or in two (the first without logits), every decoding request's logits wanted in every step,
    in an order of entries that puts the portion first, last or in the middle. NaN-poisoned pools.
    Checked against a runner without graphs and against the plain implementation."""
    from clockwork_amd.config.engine import EngineConfig
    from clockwork_amd.engine.model_runner import ModelRunner

    cfg, _, block_size = TINY_CONFIGS[name]
    gen = torch.Generator().manual_seed(45)
    vocab = cfg["vocab_size"]
    toks = {f"d{i}": torch.randint(0, vocab, (n + 40,), generator=gen).tolist() for i, n in enumerate([33, 70, 9])}
    at = {"d0": 33, "d1": 70, "d2": 9}
    steps = [{"entries": [{"id": rid, "tokens": toks[rid][:n], "want": []}], "end": []} for rid, n in at.items()]
    arrivals = [5, 5, 5, 16, 17, 30, 30, 64, 65, 100, 100, 128, 129, 200, 200, 2, 2, 2]
    for i, n in enumerate(arrivals):
        rid = f"p{i}"
        toks[rid] = torch.randint(0, vocab, (n + 40,), generator=gen).tolist()
        cuts = [n] if i % 3 else [n // 2, n - n // 2]
        if min(cuts) < 2:
            cuts = [n]
        begin = 0
        for c, size in enumerate(cuts):
            singles = []
            for d in sorted(at):
                singles.append({"id": d, "tokens": toks[d][at[d] : at[d] + 1], "want": [0]})
                at[d] += 1
            portion = {"id": rid, "tokens": toks[rid][begin : begin + size], "want": [size - 1] if c == len(cuts) - 1 else []}
            begin += size
            where = (i + c) % (len(singles) + 1)
            steps.append({"entries": singles[:where] + [portion] + singles[where:], "end": []})
        if i in (3, 9):  # this prompt goes on decoding beside the others
            at[rid] = n
        else:
            steps[-1]["end"] = [rid]
    steps[-1]["end"] = steps[-1]["end"] + [d for d in at if d not in steps[-1]["end"]]

    def runner(use_graphs):
        ecfg = EngineConfig.defaults(
            str(model_dirs[name]), dtype=dtype, block_size=block_size, num_blocks=160, enable_prefix_cache=False,
            watermark=0.0, max_model_len=512,
        )
        return ModelRunner(ecfg, cache_fill=float("nan"), use_graphs=use_graphs)

    with_graphs, eager = runner(True), runner(False)
    got_g = replay.run_trace(with_graphs, [dict(s) for s in steps])
    got_e = replay.run_trace(eager, [dict(s) for s in steps])
    captured = sorted(k[1:3] for k, v in with_graphs._graphs.items() if isinstance(v, tuple) and k[0] == "mixed")
    # up to 64 rows in all a step is padded to 16, 32 or 64 rows (4 + 12, 4 + 28, 4 + 60, 8 + 8)
    assert {(4, 12), (4, 28), (4, 60), (8, 8), (8, 128), (8, 256)} <= set(captured), f"mixed graphs captured: {captured}"
    assert got_g.keys() == got_e.keys() and len(got_g) > 100
    close = dict(rtol=2e-6, atol=2e-6) if dtype == "float32" else dict(rtol=2e-2, atol=2e-2)
    for key in got_e:
        torch.testing.assert_close(got_g[key], got_e[key], **close, msg=lambda m: f"padded graph differs from the eager step at {key}: {m}")
    model = PlainQwen2(model_dirs[name])
    ref = {k: model.logits(v) for k, v in toks.items()}
    _check(got_g, ref, dtype)


@pytest.mark.parametrize("tuned", [False, True])
def test_wide_decode_batches_of_a_large_layer_replay_as_eager(tmp_path, tuned):
    """40 requests decoding together through one layer of the 7B shape: at this width some products
    are library products inside the captured graph (also a kernel the library's tuning picked;
    the runner keeps a graph only if it holds kernel nodes alone). Every replay, with eager steps of another batch
    size and synchronisations in between, must equal the same step of a runner without graphs."""
    from clockwork_amd.weights.random_init import write_random_model
    from tests import configs

    config = configs.LAYER_7B
    model_dir = write_random_model(tmp_path / "layer7b", config, 3)
    gen = torch.Generator().manual_seed(5)
    n_req, prompt, decode = 40, 6, 7
    toks = {f"r{i}": torch.randint(0, config["vocab_size"], (prompt + decode,), generator=gen).tolist() for i in range(n_req)}
    # 40 rows a step (a graph of 48), now and then only the first 19 (one of 24): a request left
    # out of a step simply goes on later
    fixed = [{"entries": [{"id": rid, "tokens": t[:prompt], "want": []} for rid, t in toks.items()], "end": []}]
    at = {rid: prompt for rid in toks}
    for d in range(decode):
        ids = list(toks) if d % 3 != 2 else list(toks)[:19]
        fixed.append({"entries": [{"id": rid, "tokens": toks[rid][at[rid] : at[rid] + 1], "want": [0]} for rid in ids], "end": []})
        for rid in ids:
            at[rid] += 1
    pages = n_req * 2 + 4
    with_graphs = replay.make_runner(model_dir, "bfloat16", 16, pages, use_graphs=True)
    eager = replay.make_runner(model_dir, "bfloat16", 16, pages, use_graphs=False)
    if tuned:
        assert with_graphs.tune_products([48, 24]) == [48, 24]
    got_g = replay.run_trace(with_graphs, [dict(s) for s in fixed])
    got_e = replay.run_trace(eager, [dict(s) for s in fixed])
    captured = [k for k, v in with_graphs._graphs.items() if isinstance(v, tuple)]
    assert {size for size, _ in captured} == {48, 24}
    assert all(set(with_graphs.graph_nodes[k]) == {"kernel"} for k in captured)
    assert got_g.keys() == got_e.keys() and len(got_g) > 200
    scale = torch.stack(list(got_e.values())).square().mean().sqrt().item()
    for key in got_e:
        assert not torch.isnan(got_g[key]).any()
        # The graph runs the padded batch (48 or 24 rows), the eager step the live rows (40 or 19):
        # the library may take another kernel for another row count and add in another order, and
        # at this many rows the logits come out of a bfloat16 product, so a logit may differ by a
        # unit in the last place of bfloat16 (2^-8 of its value; two allowed). A replay that read
        # a stale or cleared buffer is off by the logits' own scale.
        diff = (got_g[key] - got_e[key]).abs()
        bound = 2e-2 * scale + 2.0 ** -7 * got_e[key].abs()
        assert bool((diff <= bound).all()), f"graph replay differs from the eager step at {key}: {diff.max().item()}"


@pytest.mark.parametrize("tuned", [False, True])
def test_captured_graphs_hold_kernel_nodes_only(tmp_path, tuned):
    """One layer of the 7B shape: a decode batch of 96 rows and a portion of 2048 tokens, the two
    kinds of step whose graphs capture library products (also the kernels the library's tuning
    picks). The runner walks every graph it captures and keeps it only if all its nodes are kernel
    launches; here both graphs must be kept, i.e. the library recorded no memset or copy node."""
    from clockwork_amd.config.engine import EngineConfig
    from clockwork_amd.engine.batch import StepEntry
    from clockwork_amd.engine.model_runner import ModelRunner
    from clockwork_amd.weights.random_init import write_random_model
    from tests import configs

    config = configs.LAYER_7B
    model_dir = write_random_model(tmp_path / "layer7b", config, 3)
    cfg = EngineConfig.defaults(str(model_dir), dtype="bfloat16", block_size=16, num_blocks=96 + 3 * 128 + 8,
                                enable_prefix_cache=False, watermark=0.0, max_model_len=8192,
                                max_num_batched_tokens=2048, max_num_seqs=128)
    runner = ModelRunner(cfg)
    if tuned:
        assert runner.tune_products([2048, 96]) == [2048, 96]
    gen = torch.Generator().manual_seed(5)
    long_prompt = torch.randint(0, config["vocab_size"], (3 * 2048,), generator=gen).tolist()
    runner.reserve("long", 0, 3 * 2048)
    for i in range(3):  # seen, captured, replayed
        runner.step([StepEntry("long", 2048 * i, long_prompt[2048 * i : 2048 * (i + 1)], [2047])])
    for r in range(96):
        runner.reserve(f"r{r}", 0, 3)
    for i in range(3):
        runner.step([StepEntry(f"r{r}", i, [int(long_prompt[r + i])], [0]) for r in range(96)])
    torch.cuda.synchronize()
    kept = {k: v for k, v in runner._graphs.items() if isinstance(v, tuple)}
    print({k: runner.graph_nodes[k] for k in runner.graph_nodes})
    assert set(kept) == set(runner.graph_nodes)
    assert (96, 512) in kept and any(k[0] == "portion" and k[1] == 2048 for k in kept)
    for key, kinds in runner.graph_nodes.items():
        assert set(kinds) == {"kernel"} and kinds["kernel"] > 10, f"graph {key} holds {kinds}"


def test_a_graph_with_a_memset_node_is_not_kept(model_dirs, monkeypatch):
    """A captured step in which something recorded a node that is no kernel launch (a library
    product that clears a workspace with a memset) is not kept: the runner drops the graph and
    runs that batch shape eagerly from then on, with the same logits. No memset is put under a
    capture here: the walk over the captured graph's nodes is made to report one."""
    from clockwork_amd.engine import model_runner

    name = "B"
    cfg, _, block_size = TINY_CONFIGS[name]
    toks = torch.randint(0, cfg["vocab_size"], (40,), generator=torch.Generator().manual_seed(2)).tolist()
    steps = [{"entries": [{"id": "x", "tokens": [t], "want": [0]}], "end": []} for t in toks]
    clean_runner = replay.make_runner(model_dirs[name], "float32", block_size, 8)
    clean = replay.run_trace(clean_runner, [dict(s) for s in steps])
    assert isinstance(clean_runner._graphs[(1, 512)], tuple)  # the same steps do replay a graph otherwise
    real_walk = model_runner.node_kinds
    walked = []

    def walk_that_finds_a_memset(graph):
        kinds = dict(real_walk(graph))
        walked.append(dict(kinds))
        kinds["memset"] = 1
        return kinds

    monkeypatch.setattr(model_runner, "node_kinds", walk_that_finds_a_memset)
    runner = replay.make_runner(model_dirs[name], "float32", block_size, 8)
    got = replay.run_trace(runner, [dict(s) for s in steps])
    assert len(walked) == 1 and set(walked[0]) == {"kernel"}   # captured once, never again
    assert runner._graphs[(1, 512)] == "eager" and runner.graph_nodes[(1, 512)].get("memset") == 1
    for key in clean:
        torch.testing.assert_close(got[key], clean[key], rtol=2e-6, atol=2e-6)


def test_negative_control_a_small_weight_change_breaks_the_match(model_dirs, tmp_path):
    """tests/test_hf_equivalence.py:141-153: the 1e-5 bar must bite. One q_proj row of layer 1
    moved by 2^-7 is far more than the bar allows."""
    from safetensors.torch import load_file, save_file

    name = "A"
    src = model_dirs[name]
    tensors = load_file(str(src / "model.safetensors"))
    tensors["model.layers.1.self_attn.q_proj.weight"] = tensors["model.layers.1.self_attn.q_proj.weight"].clone()
    tensors["model.layers.1.self_attn.q_proj.weight"][:8] += 2.0 ** -7
    dst = tmp_path / "perturbed"
    dst.mkdir()
    (dst / "config.json").write_text((src / "config.json").read_text())
    save_file(tensors, str(dst / "model.safetensors"))
    requests = {"r0": _requests(name)["r3"]}
    runner = replay.make_runner(dst, "float32", 16, 8)
    got = replay.run_trace(runner, replay.whole(requests))
    with pytest.raises(AssertionError):
        replay.compare(got, {"r0": _plain(name, model_dirs)["r3"]}, **TOL["float32"])


def _run_program(model_dir, dtype, steps, out, max_tokens, page=None):
    lines = [json.dumps({"step": i, **s}) for i, s in enumerate(steps)]
    proc = subprocess.run(
        [sys.executable, str(REPO / "bin" / "trace_run"), "--model", str(model_dir), "--dtype", dtype,
         "--out", str(out), "--max-tokens", str(max_tokens), *([] if page is None else ["--page", str(page)])],
        input="\n".join(lines) + "\n", capture_output=True, text=True, timeout=600,
    )
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [l for l in proc.stdout.splitlines() if l.startswith("done")] == [f"done {i}" for i in range(len(steps))]


def _read_program_output(out, steps, vocab, starts=None) -> dict:
    """{(id, position): logits row} from the <step>.f32 files; ``starts``: the position a request
    that begins with shared tokens starts at."""
    at = dict(starts or {})
    got = {}
    for i, s in enumerate(steps):
        wanted = sum(len(e["want"]) for e in s["entries"])
        if not wanted:
            assert not (out / f"{i}.f32").exists()
            continue
        rows = np.fromfile(out / f"{i}.f32", dtype="<f4").reshape(-1, vocab)
        assert rows.shape[0] == wanted
        r = 0
        for e in s["entries"]:
            first = at.get(e["id"], 0)
            for w in e["want"]:
                got[(e["id"], first + w)] = torch.from_numpy(rows[r].copy())
                r += 1
            at[e["id"]] = first + len(e["tokens"])
    return got


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_program(model_dirs, tmp_path, dtype):
    """bin/trace_run as a user runs it: JSON lines in, <step>.f32 files and 'done <step>' out;
    once with its own page size, once with pages of 8 tokens (``--page``)."""
    name = "A"
    requests = {k: v for k, v in list(_requests(name).items())[:5]}
    steps = replay.mixed(requests)
    max_tokens = 4 * 64 * -(-max(len(t) for t in requests.values()) // 64)
    out = tmp_path / "out"
    _run_program(model_dirs[name], dtype, steps, out, max_tokens, page=None if dtype == "float32" else 8)
    got = _read_program_output(out, steps, TINY_CONFIGS[name][0]["vocab_size"])
    assert len(got) == sum(len(t) for t in requests.values())
    _check(got, _plain(name, model_dirs), dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_program_with_shared_pages(model_dirs, tmp_path, dtype):
    """The program's "share" and "fork" fields: the trace of requests that hold the same pages."""
    name = "B_peaked"
    vocab = TINY_CONFIGS["B"][0]["vocab_size"]
    a = torch.randint(0, vocab, (6 * 16 + 5,), generator=torch.Generator().manual_seed(8)).tolist()
    steps, seqs, starts = replay.shared(a, vocab, 16, seed=9)
    plain = PlainQwen2(model_dirs[name])
    ref = {rid: plain.logits(toks) for rid, toks in seqs.items()}
    out = tmp_path / "out"
    _run_program(model_dirs[name], dtype, steps, out, max_tokens=4 * 128)
    got = _read_program_output(out, steps, vocab, starts)
    assert len(got) == sum(len(e["tokens"]) for s in steps for e in s["entries"])
    _check(got, ref, dtype)
