"""Decode and prefill throughput of the engine on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch B] [--layers L] [--dtype bfloat16] [--shape 1.5b]
    python bench.py --workload mixed|arrivals|agent [--shape 7b] [--requests 64]

Default workload: the layer sizes of Qwen2.5-1.5B with random weights (seed 2), bfloat16,
8 requests that each hold a 2048-token prompt, context limit 4096, pages of 16 tokens. A
"step" is one decode step of the whole batch through the engine's own loop (scheduler, step
function, sampling kernels; greedy). Prints one JSON line: ``value`` is decoded tokens a second
at the default batch; ``prefill`` is one 2048-token prompt; ``roofline`` prices the decode step
against HBM bandwidth; ``points`` holds decode at batch 1 and 64.
"""

from __future__ import annotations

import argparse
import json
import sys
import time

PEAK_HBM_GBS = 8000.0
PEAK_FLOPS = {"bfloat16": 2.5e15, "float32": 157.3e12}

QWEN25_1P5B = dict(
    model_type="qwen2", architectures=["Qwen2ForCausalLM"], vocab_size=151936, hidden_size=1536,
    num_hidden_layers=28, num_attention_heads=12, num_key_value_heads=2, intermediate_size=8960,
    rms_norm_eps=1e-6, rope_theta=1000000.0, tie_word_embeddings=True, hidden_act="silu",
    use_sliding_window=False, max_position_embeddings=32768,
)
# the other layer shapes the engine is meant for (``--shape``); the default run and the recorded
# numbers are the 1.5B shape
QWEN25_7B = dict(QWEN25_1P5B, vocab_size=152064, hidden_size=3584, num_attention_heads=28, num_key_value_heads=4,
                 intermediate_size=18944, tie_word_embeddings=False)
QWEN25_32B = dict(QWEN25_1P5B, vocab_size=152064, hidden_size=5120, num_hidden_layers=64, num_attention_heads=40,
                  num_key_value_heads=8, intermediate_size=27648, tie_word_embeddings=False)
QWEN25_0P5B = dict(QWEN25_1P5B, hidden_size=896, num_hidden_layers=24, num_attention_heads=14, num_key_value_heads=2,
                   intermediate_size=4864)
QWEN25_3B = dict(QWEN25_1P5B, hidden_size=2048, num_hidden_layers=36, num_attention_heads=16, num_key_value_heads=2,
                 intermediate_size=11008)
QWEN25_14B = dict(QWEN25_1P5B, vocab_size=152064, hidden_size=5120, num_hidden_layers=48, num_attention_heads=40,
                  num_key_value_heads=8, intermediate_size=13824, tie_word_embeddings=False)
QWEN25_72B = dict(QWEN25_1P5B, vocab_size=152064, hidden_size=8192, num_hidden_layers=80, num_attention_heads=64,
                  num_key_value_heads=8, intermediate_size=29568, tie_word_embeddings=False)
SHAPES = {"0.5b": ("Qwen2.5-0.5B", QWEN25_0P5B), "1.5b": ("Qwen2.5-1.5B", QWEN25_1P5B), "3b": ("Qwen2.5-3B", QWEN25_3B),
          "7b": ("Qwen2.5-7B", QWEN25_7B), "14b": ("Qwen2.5-14B", QWEN25_14B), "32b": ("Qwen2.5-32B", QWEN25_32B),
          "72b": ("Qwen2.5-72B", QWEN25_72B)}
PROMPT_LEN = 2048   # the prefill measurement, and the decode requests' prompts unless --prompt-len says otherwise
CONTEXT = 4096
BLOCK = 16


def _sync():
    import torch

    torch.cuda.synchronize()


def context_of(args) -> int:
    """The context limit of the run: twice the decode requests' prompts, 4096 for the recorded 2048."""
    return max(CONTEXT, 2 * getattr(args, "prompt_len", PROMPT_LEN))


def build_runner(args, prefix_cache: bool = False, max_batch: int = 0):
    from clockwork_amd.config.engine import EngineConfig
    from clockwork_amd.engine.model_runner import GRAPH_BATCH_SIZES, ModelRunner

    config = dict(SHAPES[args.shape][1])
    if args.layers is not None:
        config["num_hidden_layers"] = args.layers
    args.layers = config["num_hidden_layers"]
    # the cache holds the largest batch the run decodes: 64 for the recorded points
    max_batch = max(args.batch, 1 if getattr(args, "no_points", False) else 64, max_batch)
    context = context_of(args)
    cfg = EngineConfig.defaults(
        f"random:{SHAPES[args.shape][0].lower()}", dtype=args.dtype, max_model_len=context, block_size=BLOCK,
        num_blocks=max_batch * context // BLOCK, enable_prefix_cache=prefix_cache, watermark=0.0,
        max_num_seqs=max_batch, max_num_batched_tokens=max(PROMPT_LEN, max_batch),
        # the engine's random-weights mode: every tensor drawn from the seed by the GPU's generator
        weights="random_device", weight_seed=2,
    )
    runner = ModelRunner(cfg, config_dict=config)
    if not args.no_tune:
        # the engine's start-up option ``tune_products``: the library's fastest kernel per product shape
        runner.tune_products([PROMPT_LEN, *GRAPH_BATCH_SIZES])
    return cfg, runner


def time_decode(cfg, runner, batch: int, steps: int, warmup: int, sampling=None, prompt_len: int = PROMPT_LEN):
    """Prefill ``batch`` prompts of ``prompt_len`` tokens, then time ``steps`` decode steps.
    ``sampling``: (temperature, top_k, top_p) instead of greedy."""
    import torch

    from clockwork_amd.engine.llm_engine import LLMEngine
    from clockwork_amd.engine.sequence import SamplingParams

    engine = LLMEngine(cfg, runner=runner)
    gen = torch.Generator().manual_seed(batch)
    vocab = runner.spec.vocab_size
    temperature, top_k, top_p = sampling or (0.0, -1, 1.0)
    for i in range(batch):
        # the first requests decode while the others' prompts run, portion by portion: a margin of tokens for those steps
        portions = -(-prompt_len // cfg.scheduler.max_num_batched_tokens)
        params = SamplingParams(max_tokens=warmup + steps + 2 * batch * portions + 8, temperature=temperature, top_k=top_k,
                                top_p=top_p, seed=i, ignore_eos=True)
        engine.add_request(f"b{batch}-{i}", prompt_token_ids=torch.randint(0, vocab, (prompt_len,), generator=gen).tolist(),
                           sampling_params=params)
    while any(s.is_prefilling() or s.num_computed_tokens == 0 for s in engine.scheduler.running + engine.scheduler.waiting):
        engine.step()
    for _ in range(warmup):
        engine.step()
    _sync()
    seqs = list(engine.scheduler.running)
    assert len(seqs) == batch and all(s.num_uncomputed_tokens() == 1 for s in seqs)
    ctx_begin = sum(len(s) for s in seqs) / batch
    # the host's clock around the whole loop is the measurement; events on the GPU's queue after
    # every step give the steps' own times beside it (the notebook's method, bench_t4.ipynb:236-250)
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]
    marks[0].record()
    t0 = time.perf_counter()
    for i in range(steps):
        outs = engine.step()
        marks[i + 1].record()
        assert len(outs) == batch
    _sync()
    elapsed = time.perf_counter() - t0
    for i in range(batch):
        engine.abort_request(f"b{batch}-{i}")
    mean_ctx = ctx_begin + (steps - 1) / 2.0  # keys a request reads in the middle step
    gaps = sorted(marks[i].elapsed_time(marks[i + 1]) for i in range(steps))
    LAST_STEP_TIMES.clear()
    LAST_STEP_TIMES.update(mean=round(sum(gaps) / steps, 4), p50=round(gaps[steps // 2], 4), max=round(gaps[-1], 4))
    return elapsed, mean_ctx


# per-step times of the last ``time_decode`` run, from events on the GPU's queue (milliseconds)
LAST_STEP_TIMES: dict = {}
# how the last ``time_prefill`` chose its time, and the fastest and slowest of its runs
LAST_PREFILL_TIMES: dict = {}


def time_prefill(cfg, runner, repeats: int = 6, total: int = PROMPT_LEN):
    """Seconds for one prompt of ``total`` tokens, in portions of PROMPT_LEN tokens (one step when
    total is PROMPT_LEN, the recorded measurement): the median of ``repeats`` runs after one that
    is not counted; ``LAST_PREFILL_TIMES`` keeps the runs' best and worst beside it."""
    import torch

    from clockwork_amd.engine.batch import StepEntry

    vocab = runner.spec.vocab_size
    tokens = torch.randint(0, vocab, (total,), generator=torch.Generator().manual_seed(99)).tolist()
    runs = []
    for i in range(repeats + 1):
        _sync()
        t0 = time.perf_counter()
        for at in range(0, total, PROMPT_LEN):
            n = min(PROMPT_LEN, total - at)
            runner.reserve("prefill", at, n)
            logits = runner.step([StepEntry("prefill", at, tokens[at:at + n], [n - 1] if at + n == total else [])])
        _sync()
        dt = time.perf_counter() - t0
        runner.release("prefill")
        if i > 0:  # the first run pays for library heuristics and allocations
            runs.append(dt)
    assert logits.shape == (1, vocab)
    runs.sort()
    median = runs[len(runs) // 2] if len(runs) % 2 else 0.5 * (runs[len(runs) // 2 - 1] + runs[len(runs) // 2])
    LAST_PREFILL_TIMES.clear()
    LAST_PREFILL_TIMES.update(stat=f"median of {len(runs)} runs", best_ms=round(1e3 * runs[0], 3), worst_ms=round(1e3 * runs[-1], 3))
    return median


def run_mixed(args) -> dict:
    """A continuous batch through the whole engine: ``args.requests`` requests arrive at once,
    prompt lengths uniform in [128, 2048], half of them opening with the same 1024 tokens (the
    prefix cache serves those), prompts cut into portions under a budget of 2048 tokens a step
    beside the decoding requests, 128 greedy tokens each.

    ``--workload arrivals``: the requests come one by one instead, a new one every
    ``--arrive-every`` steps, with short prompts (uniform in [32, 512], nothing shared): most
    steps then hold one prompt beside the tokens of the requests that are decoding."""
    import torch

    from clockwork_amd.engine.llm_engine import LLMEngine
    from clockwork_amd.engine.sequence import SamplingParams

    n_req, out_len, shared = args.requests, 128, 1024
    arrivals = args.workload == "arrivals"
    shortest, longest = (32, 512) if arrivals else (128, PROMPT_LEN)
    cfg, runner = build_runner(args, prefix_cache=True, max_batch=n_req)
    vocab = runner.spec.vocab_size
    gen = torch.Generator().manual_seed(7)
    common = torch.randint(0, vocab, (shared,), generator=gen).tolist()
    prompts = []
    for i in range(n_req):
        n = int(torch.randint(shortest, longest + 1, (1,), generator=gen))
        ids = torch.randint(0, vocab, (n,), generator=gen).tolist()
        if i % 2 == 1 and n > shared:
            ids[:shared] = common
        prompts.append(ids)
    params = SamplingParams(max_tokens=out_len, temperature=0.0, ignore_eos=True)

    engine = LLMEngine(cfg, runner=runner)

    def once(tag):
        engine.prefix_cache.reset()  # a cold prefix cache: only prefixes shared within the run hit
        _sync()
        before = engine.stats()
        t0 = time.perf_counter()
        waiting = list(enumerate(prompts))
        first, arrived, done, steps = {}, {}, 0, 0
        while waiting or engine.has_unfinished_requests():
            due = len(waiting) if not arrivals else int(steps % args.arrive_every == 0)
            for i, ids in waiting[:due]:
                engine.add_request(f"{tag}-{i}", prompt_token_ids=ids, sampling_params=params)
                arrived[f"{tag}-{i}"] = time.perf_counter() - t0
            del waiting[:due]
            outs = engine.step()
            steps += 1
            now = time.perf_counter() - t0
            for o in outs:
                if o.num_generated_tokens >= 1 and o.request_id not in first:
                    first[o.request_id] = now - arrived[o.request_id]
                done += bool(o.finished)
        _sync()
        elapsed = time.perf_counter() - t0
        assert done == n_req
        after = engine.stats()
        return elapsed, steps, first, {k: after[k] - before[k] for k in ("total_cached_tokens", "num_preempted_total")}

    once("warm")  # graphs captured, library kernels chosen, prefix cache filled as in a running server
    if arrivals:
        once("warm2")  # a shape is captured when it comes the second time: steps of many shapes need two passes
    elapsed, steps, first, stats = once("run")
    n_prompt = sum(len(p) for p in prompts)
    ttft = sorted(first.values())
    return {
        "metric": f"output tok/s, {SHAPES[args.shape][0]} shape, "
                  + (f"{n_req} requests arriving one every {args.arrive_every} steps" if arrivals
                     else f"continuous batch of {n_req} requests"),
        "value": round(n_req * out_len / elapsed, 1),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": steps,
        "warmup": 0,
        "ms_per_step": round(1e3 * elapsed / steps, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
        "data": "synthetic: uniform random token ids, random weights (seed 2)",
        "seconds": round(elapsed, 4),
        "prompt_tokens": n_prompt,
        "prompt_tokens_from_prefix_cache": stats["total_cached_tokens"],
        "all_tokens_per_s": round((n_prompt + n_req * out_len) / elapsed, 1),
        "first_token_ms": {"p50": round(1e3 * ttft[len(ttft) // 2], 2), "max": round(1e3 * ttft[-1], 2)},
        "preempted": stats["num_preempted_total"],
        "config": {
            "model": f"{SHAPES[args.shape][0]} shape (random weights)",
            "layers": args.layers,
            "layers_of_full_model": SHAPES[args.shape][1]["num_hidden_layers"],
            "requests": n_req,
            "prompt_len": "uniform 32..512" if arrivals else "uniform 128..2048, every second one shares its first 1024 tokens",
            "output_len": out_len,
            "token_budget": PROMPT_LEN,
            "seq_len": CONTEXT,
            "block_size": BLOCK,
            "sampling": "greedy",
            "parallelism": "single GPU",
        },
    }


def run_agent(args) -> dict:
    """Sessions of several turns over a shared opening, the shape of traffic that the reference's
    agent traces model (docs/results.md: a system prompt of 1024 tokens that every session opens
    with, 4 to 8 turns a session): turn t's prompt is the opening, the session's earlier turns
    (their inputs and the generated answers) and 64 to 256 new tokens; 32 to 96 greedy tokens are
    generated a turn. ``--concurrency`` sessions run at a time, each sending its next turn when the
    last one is finished; ``--requests`` sessions in all. With the prefix cache a turn computes its
    new tokens only; ``--no-prefix-cache`` runs the same traffic without it."""
    import torch

    from clockwork_amd.engine.llm_engine import LLMEngine
    from clockwork_amd.engine.sequence import SamplingParams

    n_sessions, opening = args.requests, args.opening
    args.prompt_len = max(args.prompt_len, opening)  # the context is sized for twice this
    cfg, runner = build_runner(args, prefix_cache=not args.no_prefix_cache, max_batch=max(args.concurrency, 8))
    vocab = runner.spec.vocab_size
    gen = torch.Generator().manual_seed(11)
    common = torch.randint(0, vocab, (opening,), generator=gen).tolist()
    sessions = []
    for _ in range(n_sessions):
        turns = int(torch.randint(4, 9, (1,), generator=gen))
        sessions.append([torch.randint(0, vocab, (int(torch.randint(64, 257, (1,), generator=gen)),), generator=gen).tolist()
                         for _ in range(turns)])
    # answers of 32 to 96 tokens, so that the sessions do not fall into step with one another
    answer = [[int(torch.randint(32, 97, (1,), generator=gen)) for _ in turns] for turns in sessions]
    engine = LLMEngine(cfg, runner=runner)

    def once(tag):
        engine.prefix_cache.reset()
        _sync()
        before = engine.stats()
        t0 = time.perf_counter()
        history = {}   # session -> tokens so far
        turn_of = {}   # session -> index of the turn that is running
        sent, first = {}, []
        queue = list(range(n_sessions))
        prompt_tokens = outputs = steps = 0

        def send(i):
            nonlocal prompt_tokens
            t = turn_of[i]
            history[i] = history[i] + sessions[i][t]
            rid = f"{tag}-{i}-{t}"
            engine.add_request(rid, prompt_token_ids=history[i],
                               sampling_params=SamplingParams(max_tokens=answer[i][t], temperature=0.0, ignore_eos=True))
            sent[rid] = time.perf_counter()
            prompt_tokens += len(history[i])

        running = 0
        while queue or running:
            while queue and running < args.concurrency:
                i = queue.pop(0)
                history[i], turn_of[i] = list(common), 0
                send(i)
                running += 1
            outs = engine.step()
            steps += 1
            now = time.perf_counter()
            for o in outs:
                if o.num_generated_tokens == 1:
                    first.append(now - sent[o.request_id])
                if o.finished:
                    outputs += o.num_generated_tokens
                    i = int(o.request_id.split("-")[1])
                    history[i] = history[i] + list(o.token_ids)
                    turn_of[i] += 1
                    if turn_of[i] < len(sessions[i]):
                        send(i)
                    else:
                        running -= 1
        _sync()
        elapsed = time.perf_counter() - t0
        after = engine.stats()
        cached = after["total_cached_tokens"] - before["total_cached_tokens"]
        return elapsed, steps, first, prompt_tokens, outputs, cached

    once("warm")   # graphs captured, the library's kernels chosen
    once("warm2")  # a shape is captured when it comes the second time
    elapsed, steps, first, prompt_tokens, outputs, cached = once("run")
    first.sort()
    return {
        "metric": f"output tok/s, {SHAPES[args.shape][0]} shape, {n_sessions} sessions of 4 to 8 turns, {args.concurrency} at a time",
        "value": round(outputs / elapsed, 1),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": steps,
        "warmup": 0,
        "ms_per_step": round(1e3 * elapsed / steps, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
        "data": "synthetic: uniform random token ids, random weights (seed 2)",
        "seconds": round(elapsed, 4),
        "turns": len(first),
        "prompt_tokens": prompt_tokens,
        "prompt_tokens_from_prefix_cache": cached,
        "hit_rate": round(cached / max(prompt_tokens, 1), 3),
        "first_token_ms": {"p50": round(1e3 * first[len(first) // 2], 2), "p99": round(1e3 * first[min(len(first) - 1, int(0.99 * len(first)))], 2)},
        "config": {
            "model": f"{SHAPES[args.shape][0]} shape (random weights)",
            "layers": args.layers,
            "layers_of_full_model": SHAPES[args.shape][1]["num_hidden_layers"],
            "sessions": n_sessions,
            "concurrency": args.concurrency,
            "opening": opening,
            "turn_input": "uniform 64..256",
            "output_len": "uniform 32..96",
            "prefix_cache": not args.no_prefix_cache,
            "token_budget": PROMPT_LEN,
            "seq_len": context_of(args),
            "block_size": BLOCK,
            "sampling": "greedy",
            "parallelism": "single GPU",
        },
    }


def measure_peaks() -> dict:
    """What this card reaches on the two plainest workloads, beside the published peaks the
    fractions are priced against: a device-to-device copy of 2 GiB (bytes read + written) and the
    library's bfloat16 product of 8192 x 8192 x 8192."""
    import torch

    def best_of(fn, n=5):
        fn()
        best = None
        for _ in range(n):
            _sync()
            t0 = time.perf_counter()
            fn()
            _sync()
            dt = time.perf_counter() - t0
            best = dt if best is None else min(best, dt)
        return best

    src = torch.empty(1 << 30, dtype=torch.int16, device="cuda").zero_()
    dst = torch.empty_like(src)
    t_copy = best_of(lambda: dst.copy_(src))
    n = 8192
    a = torch.randn(n, n, device="cuda", dtype=torch.bfloat16)
    b = torch.randn(n, n, device="cuda", dtype=torch.bfloat16)
    t_mm = best_of(lambda: torch.mm(a, b.t()))
    return {
        "copy_GBps": round(2 * src.numel() * 2 / t_copy / 1e9, 1),
        "copy_frac_of_hbm_peak": round(2 * src.numel() * 2 / t_copy / 1e9 / PEAK_HBM_GBS, 4),
        "bf16_product_TFLOPs": round(2 * n ** 3 / t_mm / 1e12, 1),
        "bf16_product_frac_of_mfma_peak": round(2 * n ** 3 / t_mm / PEAK_FLOPS["bfloat16"], 4),
    }


# The reference's only kernel-level figures: its paged decode attention alone, on its own card
# (/root/reference/docs/results.md:83-94: Tesla T4, float16, 12 query heads on 2 key/value heads,
# head size 128, pages of 16; milliseconds by (batch, context)).
REFERENCE_DECODE_ATTENTION_MS = {
    (1, 128): 0.0607, (1, 512): 0.1602, (1, 2048): 0.6219, (4, 128): 0.0737, (4, 512): 0.2735, (4, 2048): 0.5802,
    (16, 128): 0.0979, (16, 512): 0.4182, (16, 2048): 1.4058, (64, 128): 0.4079, (64, 512): 1.4359, (64, 2048): 5.3783,
}


def measure_decode_attention_grid() -> dict:
    """The engine's attention part alone on batches of single tokens, over the grid of batch sizes
    and context lengths that the reference times its decode kernel on (its method: 10 warm-up
    calls, then 50 timed ones, /root/reference/notebooks/bench_t4.ipynb:236-250; here the 50 calls
    are one captured graph, so the time is the kernels', the merge of the key splits included).
    Pages lie in random order; bytes are the keys and values read."""
    import torch

    from clockwork_amd.engine.batch import StepContext
    from clockwork_amd.parts.attention import PagedAttention
    from clockwork_amd.parts.specs import AttentionSpec

    dev = torch.device("cuda:0")
    nh, nkv, hd, bs = 12, 2, 128, BLOCK
    part = PagedAttention(AttentionSpec(hidden_size=nh * hd, num_heads=nh, num_kv_heads=nkv, head_dim=hd,
                                        qkv_bias=False, out_bias=False, scale=hd ** -0.5))
    part.dtype = torch.bfloat16
    units = torch.cuda.get_device_properties(dev).multi_processor_count
    grid = {}
    for (batch, context), ref_ms in REFERENCE_DECODE_ATTENTION_MS.items():
        pages_each = -(-context // bs)
        pages = batch * pages_each
        gen = torch.Generator(device="cpu").manual_seed(batch * 100003 + context)
        k = torch.randn((pages, bs, nkv, hd), generator=gen).to(dev, torch.bfloat16)
        v = torch.randn((pages, bs, nkv, hd), generator=gen).to(dev, torch.bfloat16)
        q = torch.randn((batch, nh * hd), generator=gen).to(dev, torch.bfloat16)
        ctx = StepContext()
        ctx.device, ctx.block_size, ctx.num_compute_units = dev, bs, units
        ctx.num_tokens = ctx.num_requests = batch
        ctx.h_q_lens, ctx.h_ctx_lens = [1] * batch, [context] * batch
        ctx.block_tables = [torch.randperm(pages, generator=gen).to(dev, torch.int32).view(batch, pages_each)]
        ctx.ctx_lens = torch.full((batch,), context, dtype=torch.int32, device=dev)
        ctx.cu_q = torch.arange(batch + 1, dtype=torch.int32, device=dev)
        cache = argparse.Namespace(k=k, v=v, group=0, block_size=bs)
        part.prepare(ctx)
        for _ in range(10):
            part.attend(q, ctx, cache)
        _sync()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            for _ in range(50):
                part.attend(q, ctx, cache)
        graph.replay()
        _sync()
        begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        begin.record()
        graph.replay()
        end.record()
        end.synchronize()
        ms = begin.elapsed_time(end) / 50
        plan = part._plan(ctx, torch.bfloat16)
        read = 2 * batch * context * nkv * hd * 2
        grid[f"batch{batch}_ctx{context}"] = {"ms": round(ms, 5), "reference_t4_ms": ref_ms, "key_splits": plan.decode_splits,
                                              "GB_per_s": round(read / ms / 1e6, 1)}
    return {"metric": "paged decode attention alone, 12 query heads on 2 key/value heads, head size 128, pages of 16",
            "unit": "ms", "dtype": "bf16", "stat": "mean of 50 calls in one graph after 10 warm-up calls",
            "reference": "Tesla T4, float16 (docs/results.md:83-94 of the reference): other hardware, for orientation",
            "grid": grid}


def prefill_flops(spec, model, T: int) -> float:
    """2 * T * (matrix parameters of the layers) + causal attention + one row of the output head."""
    layer_params = 0
    for name, t in model.params.items():
        if name.startswith("layers.") and t.dim() == 2:
            layer_params += t.numel()
    info = spec.info
    attn = 4.0 * info["head_dim"] * info["heads"] * (T * (T + 1) / 2.0) * info["layers"]
    head = 2.0 * info["hidden"] * info["vocab"]
    return 2.0 * T * layer_params + attn + head


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--prompt-len", type=int, default=PROMPT_LEN,
                    help="tokens each decode request holds before it decodes (the recorded benchmark: 2048)")
    ap.add_argument("--layers", type=int, default=None, help="fewer layers than the shape has (both numbers are recorded)")
    ap.add_argument("--shape", default="1.5b", choices=sorted(SHAPES), help="layer sizes: the 1.5B shape is the recorded benchmark")
    ap.add_argument("--dtype", default="bfloat16", choices=("bfloat16", "float32"))
    ap.add_argument("--no-points", action="store_true", help="skip the batch 1 / 64 points and the prefill")
    ap.add_argument("--no-tune", action="store_true", help="leave the matrix library's kernel choice at its default")
    ap.add_argument("--only-prefill", action="store_true", help="run the prefill alone: 2048 tokens, or --prompt-len tokens in portions of 2048")
    ap.add_argument("--arrive-every", type=int, default=4, help="--workload arrivals: steps between two requests")
    ap.add_argument("--workload", default="decode", choices=("decode", "mixed", "arrivals", "agent"),
                    help="decode: the recorded benchmark; mixed: a continuous batch of --requests prompts of mixed lengths; "
                         "arrivals: short prompts coming one by one; agent: sessions of several turns over a shared opening")
    ap.add_argument("--concurrency", type=int, default=8, help="--workload agent: sessions that run at a time")
    ap.add_argument("--opening", type=int, default=1024, help="--workload agent: tokens that every session opens with")
    ap.add_argument("--no-prefix-cache", action="store_true", help="--workload agent: the same traffic without the prefix cache")
    ap.add_argument("--requests", type=int, default=64)
    ap.add_argument("--peaks", action="store_true", help="measure a device copy and a large library product instead")
    ap.add_argument("--decode-attention-grid", action="store_true",
                    help="time the attention part alone over the reference's grid of batch sizes and context lengths instead")
    ap.add_argument("--temperature", type=float, default=0.0, help="sample instead of the greedy decoding of the recorded benchmark")
    ap.add_argument("--top-k", type=int, default=-1)
    ap.add_argument("--top-p", type=float, default=1.0)
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU: this engine has no multi-GPU path (asked for --gpus {args.gpus})")
        return 2

    import torch

    if args.peaks:
        print(json.dumps(measure_peaks()))
        return 0
    if args.decode_attention_grid:
        print(json.dumps(measure_decode_attention_grid()))
        return 0
    if args.workload == "agent":
        print(json.dumps(run_agent(args)))
        return 0
    if args.workload in ("mixed", "arrivals"):
        print(json.dumps(run_mixed(args)))
        return 0
    cfg, runner = build_runner(args)
    if args.only_prefill:
        t = time_prefill(cfg, runner, total=args.prompt_len)
        print(json.dumps({"prefill_ms": round(1e3 * t, 3), "tokens": args.prompt_len, "portion": PROMPT_LEN,
                          "tokens_per_s": round(args.prompt_len / t, 1), **LAST_PREFILL_TIMES}))
        return 0
    sampling = (args.temperature, args.top_k, args.top_p) if args.temperature > 0 else None
    elapsed, mean_ctx = time_decode(cfg, runner, args.batch, args.steps, args.warmup, sampling, args.prompt_len)
    value = args.batch * args.steps / elapsed
    ms = 1e3 * elapsed / args.steps
    step_times = dict(LAST_STEP_TIMES)
    step_bytes = runner.model.weight_bytes_per_step() + args.batch * mean_ctx * runner.pools.kv_bytes_per_token()
    achieved = step_bytes / (elapsed / args.steps) / 1e9

    record = {
        "metric": f"decode tok/s, {SHAPES[args.shape][0]} shape, batch {args.batch}, {args.prompt_len}-token prompts",
        "value": round(value, 1),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms, 4),
        "ms_per_step_by_gpu_events": step_times,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
        "data": "synthetic: uniform random token ids, random weights (seed 2)",
        "config": {
            "model": f"{SHAPES[args.shape][0]} shape (random weights)",
            "layers": args.layers,
            "layers_of_full_model": SHAPES[args.shape][1]["num_hidden_layers"],
            "hidden": runner.spec.info["hidden"],
            "heads": runner.spec.info["heads"],
            "kv_heads": runner.spec.info["kv_heads"],
            "head_dim": runner.spec.info["head_dim"],
            "intermediate": runner.spec.info["intermediate"],
            "vocab": runner.spec.info["vocab"],
            "tied_embeddings": runner.spec.info["tied"],
            "global_batch": args.batch,
            "prompt_len": args.prompt_len,
            "seq_len": context_of(args),
            "block_size": BLOCK,
            "sampling": "greedy" if sampling is None else f"temperature {args.temperature} top_k {args.top_k} top_p {args.top_p}",
            "parallelism": "single GPU",
        },
        "roofline": {
            "bound": "hbm",
            "achieved": round(achieved, 1),
            "peak": PEAK_HBM_GBS,
            "unit": "GB/s",
            "frac": round(achieved / PEAK_HBM_GBS, 4),
        },
    }
    # what the start-up's measurements chose for this model's shapes (``tune_products``)
    products = runner.products
    record["tuned"] = {
        "gate_up_wide_tile": {f"{n}x{k}": bool(v) for (n, k), v in products.swiglu_choices.items()},
        "decode_k_splits": {f"{n}x{k}": int(v) for (n, k), v in products.k_split_choices.items()},
        "prefill_k_runs": {f"{n}x{k}": int(v) for (n, k), v in products.wide_partial_choices.items()},
    }
    if not args.no_points:
        t = time_prefill(cfg, runner)
        flops = prefill_flops(runner.spec, runner.model, PROMPT_LEN)
        record["prefill"] = {
            "value": round(PROMPT_LEN / t, 1),
            "tokens": PROMPT_LEN,
            "ms": round(1e3 * t, 3),
            "frac": round(flops / t / PEAK_FLOPS[args.dtype], 4),
            **LAST_PREFILL_TIMES,
        }
        points = {}
        for b in (1, 64):
            e, _ = time_decode(cfg, runner, b, args.steps, args.warmup, sampling, args.prompt_len)
            points[f"decode_b{b}"] = round(b * args.steps / e, 1)
        record["points"] = points
    print(json.dumps(record))
    return 0


if __name__ == "__main__":
    sys.exit(main())
