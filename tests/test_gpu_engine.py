"""Generation through the entry point: scheduler, step function, sampling, prefix cache and
preemption together, against the plain implementation and against each request run alone."""

import pytest
import torch

from clockwork_amd.config.engine import EngineConfig
from clockwork_amd.engine.sequence import SamplingParams
from tests.configs import TINY_CONFIGS
from tests.plain.qwen2_plain import PlainQwen2

pytestmark = pytest.mark.gpu


def engine(model_dir, **overrides):
    from clockwork_amd.engine.llm_engine import LLMEngine

    defaults = dict(dtype="float32", block_size=4, num_blocks=128, watermark=0.0)
    defaults.update(overrides)
    return LLMEngine(EngineConfig.defaults(str(model_dir), **defaults))


def prompts_for(name, lengths, seed=0):
    vocab = TINY_CONFIGS[name][0]["vocab_size"]
    gen = torch.Generator().manual_seed(seed)
    return [torch.randint(0, vocab, (n,), generator=gen).tolist() for n in lengths]


def greedy(n):
    return SamplingParams(max_tokens=n, temperature=0.0, ignore_eos=True)


@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_greedy_generation_equals_the_plain_implementation(model_dirs, name):
    # prompt lengths 1, 3, 9, 17 and 24 greedy tokens: tests/test_hf_equivalence.py:14,17,108-113
    prompts = prompts_for(name, [1, 3, 9, 17])
    plain = PlainQwen2(model_dirs[name])
    outs = engine(model_dirs[name]).generate(prompts, greedy(24))
    for prompt, out in zip(prompts, outs):
        assert out.token_ids == plain.greedy(prompt, 24)
        assert out.finished and out.finish_reason == "length" and out.num_generated_tokens == 24
        assert out.prompt_token_ids == prompt


def test_bfloat16_generation_follows_the_plain_implementation(model_dirs):
    name = "B"
    prompts = prompts_for(name, [5, 40])
    plain = PlainQwen2(model_dirs[name])
    outs = engine(model_dirs[name], dtype="bfloat16").generate(prompts, greedy(8))
    for prompt, out in zip(prompts, outs):
        want = plain.greedy(prompt, 8)
        # bfloat16 may flip a near-tie; up to the first flip the tokens agree, and a flip must be a near-tie
        for i, (a, b) in enumerate(zip(out.token_ids, want)):
            if a != b:
                row = plain.logits(prompt + want[:i])[-1]
                assert float(row[b] - row[a]) < 0.05
                break


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_steps_decided_one_step_ahead_change_nothing(model_dirs, dtype):
    """Requests that end at different times (lengths, an end-of-sequence token), one arriving in
    the middle and one aborted: with and without looking ahead the same tokens come out, and the
    plain decode stretches do run from schedules made ahead."""
    from clockwork_amd.engine.llm_engine import LLMEngine

    name = "A"
    prompts = prompts_for(name, [6, 11, 3, 20, 8], seed=4)
    lengths = [30, 7, 19, 12, 25]

    def session(lookahead: bool):
        eng = LLMEngine(EngineConfig.defaults(str(model_dirs[name]), dtype=dtype, block_size=4, num_blocks=256,
                                              watermark=0.0, lookahead=lookahead, enable_prefix_cache=False))
        finals = {}
        for i in range(3):
            eng.add_request(f"r{i}", prompt_token_ids=prompts[i], sampling_params=greedy(lengths[i]))
        step = 0
        while eng.has_unfinished_requests():
            if step == 9:
                eng.add_request("r3", prompt_token_ids=prompts[3], sampling_params=greedy(lengths[3]))
                eng.add_request("r4", prompt_token_ids=prompts[4], sampling_params=greedy(lengths[4]))
            if step == 15:
                eng.abort_request("r4")
            for out in eng.step():
                if out.finished:
                    finals[out.request_id] = out.token_ids
            step += 1
        assert eng.manager.min_free_blocks() == eng.manager.num_blocks
        return finals, eng.stats()["lookahead_steps"], step

    with_ahead, used, steps_a = session(True)
    without, unused, steps_b = session(False)
    assert with_ahead == without and steps_a == steps_b
    assert unused == 0 and used >= 10
    assert sorted(with_ahead) == ["r0", "r1", "r2", "r3"] and [len(with_ahead[f"r{i}"]) for i in range(4)] == lengths[:4]
    # a stop token ends a request in the middle of a stretch: the step made ahead is dropped
    stop = with_ahead["r0"][10]
    eng = LLMEngine(EngineConfig.defaults(str(model_dirs[name]), dtype=dtype, block_size=4, num_blocks=256, watermark=0.0,
                                          enable_prefix_cache=False))
    eng.add_request("s", prompt_token_ids=prompts[0],
                    sampling_params=SamplingParams(max_tokens=30, temperature=0.0, ignore_eos=True, stop_token_ids=[stop]))
    eng.add_request("t", prompt_token_ids=prompts[1], sampling_params=greedy(20))
    finals = {}
    while eng.has_unfinished_requests():
        for out in eng.step():
            if out.finished:
                finals[out.request_id] = (out.token_ids, out.finish_reason)
    first = with_ahead["r0"].index(stop)
    assert finals["s"] == (with_ahead["r0"][: first + 1], "stop")
    assert len(finals["t"][0]) == 20 and eng.stats()["lookahead_steps"] > 0
    assert eng.manager.min_free_blocks() == eng.manager.num_blocks


def test_eight_staggered_requests_equal_each_alone(model_dirs):
    # tests/test_llm_engine.py:94-131: a budget of 32 tokens forces portions and mixed steps
    name = "A"
    prompts = prompts_for(name, [12, 30, 7, 45, 3, 19, 26, 50], seed=3)
    alone = [engine(model_dirs[name]).generate([p], greedy(10))[0].token_ids for p in prompts[:3]]
    plain = PlainQwen2(model_dirs[name])
    e = engine(model_dirs[name], max_num_batched_tokens=32, enable_prefix_cache=False)
    finals = {}
    pending = list(enumerate(prompts))
    for step in range(400):
        if pending and step % 2 == 0:
            i, p = pending.pop(0)
            e.add_request(f"r{i}", prompt_token_ids=p, sampling_params=greedy(10))
        for out in e.step():
            if out.finished:
                finals[out.request_id] = out.token_ids
        if not pending and not e.has_unfinished_requests():
            break
    assert len(finals) == 8
    for i, p in enumerate(prompts):
        assert finals[f"r{i}"] == plain.greedy(p, 10), f"request {i}"
    assert [finals[f"r{i}"] for i in range(3)] == alone
    assert e.manager.min_free_blocks() == 128


def follows_plain(plain, prompt, tokens, stops=()) -> None:
    """``tokens`` are the plain implementation's greedy tokens; in bfloat16, up to the first place
    where rounding flips a near-tie: there the plain logits of the two tokens must lie within a
    twentieth of the logits' scale (a wrong key or page moves them by the scale itself)."""
    ids = list(prompt)
    for i, token in enumerate(tokens):
        row = plain.logits(ids)[-1]
        best = int(row.argmax())
        if token != best:
            gap, scale = float(row[best] - row[token]), float(row.square().mean().sqrt())
            assert gap < 0.05 * scale, f"token {i}: {token} instead of {best}, {gap:.3e} apart at a scale of {scale:.3e}"
            return
        ids.append(token)
        if token in stops:
            assert i == len(tokens) - 1
            return


# tests/test_llm_engine.py:134-165: lengths [12, 10, 15, 8], pages of 4 -> cached [8, 8, 12, 4];
# the same with pages of 8 on the other model
PREFIX_CASES = {"A": (4, [12, 10, 15, 8], [8, 8, 12, 4]), "B_peaked": (8, [24, 20, 30, 16], [16, 16, 24, 8])}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(PREFIX_CASES))
def test_prefix_cache_second_pass_is_identical_and_counts_cached_tokens(model_dirs, name, dtype):
    block_size, lengths, cached = PREFIX_CASES[name]
    prompts = prompts_for(name[0], lengths, seed=5)
    e = engine(model_dirs[name], dtype=dtype, block_size=block_size)
    first = e.generate(prompts, greedy(6))
    assert [o.num_cached_tokens for o in first] == [0, 0, 0, 0]
    second = e.generate(prompts, greedy(6))   # reads pages that the first pass's requests wrote
    assert [o.num_cached_tokens for o in second] == cached
    assert e.stats()["prefix_cache_hit_tokens"] == sum(cached)
    off = engine(model_dirs[name], dtype=dtype, block_size=block_size, enable_prefix_cache=False).generate(prompts, greedy(6))
    plain = PlainQwen2(model_dirs[name])
    if dtype == "float32":
        assert [o.token_ids for o in second] == [o.token_ids for o in first] == [o.token_ids for o in off]
        assert [o.token_ids for o in first] == [plain.greedy(p, 6) for p in prompts]
    else:
        # a hit runs the rest of the prompt as a step of another shape: other kernels, other rounding
        for outs in (first, second, off):
            for prompt, o in zip(prompts, outs):
                follows_plain(plain, prompt, o.token_ids)


def test_shared_prefix_accounting(model_dirs):
    # tests/test_llm_engine.py:168-200: four 19-token prompts sharing 16 tokens, one at a time
    name = "A"
    shared = prompts_for(name, [16], seed=9)[0]
    prompts = [shared + [i + 1, i + 2, i + 3] for i in range(4)]
    e = engine(model_dirs[name])
    plain = PlainQwen2(model_dirs[name])
    for p in prompts:
        out = e.generate([p], greedy(4))[0]
        assert out.token_ids == plain.greedy(p, 4)
    s = e.stats()
    assert (s["prefix_cache_queries"], s["prefix_cache_prompt_tokens"], s["prefix_cache_hit_tokens"]) == (4, 76, 48)
    assert s["prefix_cache_hit_rate"] == 48 / 76


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,block_size", [("A", 4), ("B_peaked", 8)])
def test_preemption_leaves_outputs_unchanged(model_dirs, name, block_size, dtype):
    # tests/test_llm_engine.py:203-219: 8 pages of 4, three requests of 8 + 8 tokens (pages of 8: 16 + 16)
    n = 2 * block_size
    prompts = prompts_for(name[0], [n, n, n], seed=11)
    plain = PlainQwen2(model_dirs[name])
    e = engine(model_dirs[name], dtype=dtype, block_size=block_size, num_blocks=8, enable_prefix_cache=False)
    outs = e.generate(prompts, greedy(n))
    assert e.stats()["num_preempted_total"] > 0
    for p, o in zip(prompts, outs):
        if dtype == "float32":
            assert o.token_ids == plain.greedy(p, n)
        else:
            assert len(o.token_ids) == n
            follows_plain(plain, p, o.token_ids)
    assert e.manager.min_free_blocks() == 8


def test_a_request_that_can_never_fit_is_an_error(model_dirs):
    e = engine(model_dirs["A"], num_blocks=2, enable_prefix_cache=False)
    e.add_request("big", prompt_token_ids=list(range(12)))
    with pytest.raises(RuntimeError, match="cannot be admitted"):
        e.step()


def test_seeded_sampling_is_reproducible_and_seeds_differ(model_dirs):
    # tests/test_llm_engine.py:222-236
    name = "B"
    prompt = prompts_for(name, [9], seed=2)

    def run(seed, **kw):
        params = SamplingParams(max_tokens=12, temperature=1.5, seed=seed, ignore_eos=True, **kw)
        return engine(model_dirs[name]).generate(prompt, params)[0].token_ids

    assert run(1) == run(1)
    assert run(1) != run(2)
    assert run(1, top_k=1) == PlainQwen2(model_dirs[name]).greedy(prompt[0], 12)  # tests/test_server.py:323
    # a request samples the same tokens alone and in a crowd
    e = engine(model_dirs[name], max_num_batched_tokens=16)
    crowd = prompts_for(name, [20, 5, 33], seed=4)
    e.add_request("x", prompt_token_ids=prompt[0], sampling_params=SamplingParams(max_tokens=12, temperature=1.5, seed=1, ignore_eos=True))
    for i, p in enumerate(crowd):
        e.add_request(f"c{i}", prompt_token_ids=p, sampling_params=SamplingParams(max_tokens=9, temperature=0.7, seed=i, ignore_eos=True))
    got = None
    while e.has_unfinished_requests():
        for out in e.step():
            if out.finished and out.request_id == "x":
                got = out.token_ids
    assert got == run(1)


def test_the_stated_sampling_workload_token_by_token_against_the_plain_sampler(model_dirs):
    """The tiny model B's workload as the benchmark description states it: five prompts of 1, 9,
    40, 64 and 100 tokens, two of which share their first 32, at most 24 tokens a step, twelve
    tokens each at temperature 0.8; seeds given for three requests, left to the engine's for two;
    so few pages that a request is preempted and computed again. In float32 every sampled token
    is the one the plain sampler draws (clockwork/engine/model_runner.py:134-164: logits /
    temperature, softmax, one draw) from the plain logits of the tokens so far with the request's
    n-th uniform number, n being the outputs it has (a preempted request draws the same numbers
    again); draws that land within 1e-4 of an interval's edge are not judged."""
    from tests.plain import qwen2_plain as plain_sampling

    name, vocab = "B", TINY_CONFIGS["B"][0]["vocab_size"]
    gen = torch.Generator().manual_seed(77)
    draw = lambda n: torch.randint(0, vocab, (n,), generator=gen).tolist()
    shared = draw(32)
    prompts = [draw(1), draw(9), draw(40), shared + draw(32), shared + draw(68)]
    assert [len(p) for p in prompts] == [1, 9, 40, 64, 100]
    seeds = [21, None, 23, None, 25]
    plain = PlainQwen2(model_dirs[name])

    def run(num_blocks):
        e = engine(model_dirs[name], dtype="float32", block_size=8, num_blocks=num_blocks, max_num_batched_tokens=24,
                   seed=5, enable_prefix_cache=True)

        def add(i):
            e.add_request(f"s{i}", prompt_token_ids=prompts[i],
                          sampling_params=SamplingParams(max_tokens=12, temperature=0.8, seed=seeds[i], ignore_eos=True))

        for i in range(4):
            add(i)
        finals = {}
        late = [4]   # the longest prompt arrives once the prompt whose beginning it shares has been computed
        while e.has_unfinished_requests() or late:
            if late and (e._seqs["s3"].output_token_ids if "s3" in e._seqs else True):
                add(late.pop())
            for out in e.step():
                if out.finished:
                    finals[out.request_id] = out
        return finals, e.stats()

    def judge(finals):
        judged = 0
        for i, (prompt, seed) in enumerate(zip(prompts, seeds)):
            tokens = finals[f"s{i}"].token_ids
            assert len(tokens) == 12
            rows = plain.logits(prompt + tokens)[len(prompt) - 1 : -1]    # the logits each output token was drawn from
            for n, token in enumerate(tokens):
                probs = plain_sampling.sampling_probs(rows[n], 0.8)
                want, margin = plain_sampling.draw(probs, plain_sampling.uniform01(5 if seed is None else seed, n))
                if margin > 1e-4:
                    judged += 1
                    assert token == want, f"request s{i}, output {n}: sampled {token}, the plain sampler draws {want}"
        return judged

    # the same workload on ever fewer pages: roomy, then so tight that requests are preempted (the
    # five hold 36 pages at their ends, the longest prompt alone 13)
    preempted = hits = 0
    for num_blocks in (64, 30, 26, 22, 18):
        finals, stats = run(num_blocks)
        assert judge(finals) >= 40   # of 60: near-uniform probabilities of 1e-3 leave a fifth within 1e-4 of an edge
        preempted += stats["num_preempted_total"]
        hits += stats["prefix_cache_hit_tokens"]
        print(f"{num_blocks} pages: preempted {stats['num_preempted_total']}, prefix hits {stats['prefix_cache_hit_tokens']} tokens")
    assert preempted > 0, "no pool was small enough to preempt a request"
    assert hits >= 32


def test_finish_rules(model_dirs):
    # tests/test_llm_engine.py:239-296
    name = "A"
    prompt = prompts_for(name, [10], seed=6)[0]
    free = engine(model_dirs[name]).generate([prompt], greedy(8))[0].token_ids
    stop_at = free[3]
    first = free.index(stop_at)
    out = engine(model_dirs[name]).generate([prompt], SamplingParams(max_tokens=8, stop_token_ids=[stop_at]))[0]
    assert out.finish_reason == "stop" and out.token_ids == free[: first + 1]  # the stop token stays in the ids
    cfg_eos = dict(TINY_CONFIGS[name][0], eos_token_id=stop_at)
    from clockwork_amd.engine.llm_engine import LLMEngine

    e = LLMEngine(EngineConfig.defaults(str(model_dirs[name]), block_size=4, num_blocks=64), config_dict=cfg_eos)
    assert e.generate([prompt], SamplingParams(max_tokens=8))[0].token_ids == free[: first + 1]
    e = LLMEngine(EngineConfig.defaults(str(model_dirs[name]), block_size=4, num_blocks=64), config_dict=cfg_eos)
    assert e.generate([prompt], SamplingParams(max_tokens=8, ignore_eos=True))[0].token_ids == free
    # max_model_len 16 with a 10-token prompt: 6 tokens, "length"
    out = engine(model_dirs[name], max_model_len=16).generate([prompt], greedy(50))[0]
    assert out.num_generated_tokens == 6 and out.finish_reason == "length"
    with pytest.raises(ValueError, match="leaves no room"):
        engine(model_dirs[name], max_model_len=10).add_request("x", prompt_token_ids=prompt)


class IntTokenizer:
    """Token i is the text "<i>" (tests/test_llm_engine.py:17-27 uses a fake of this kind)."""

    eos_token_id = None

    def encode(self, text):
        return [int(t) for t in text.replace(">", "").split("<") if t]

    def decode(self, ids, skip_special_tokens=True):
        return "".join(f"<{i}>" for i in ids)


def test_text_prompts_and_stop_strings_need_and_use_a_tokenizer(model_dirs):
    from clockwork_amd.engine.llm_engine import LLMEngine

    name = "A"
    prompt = prompts_for(name, [6], seed=8)[0]
    cfg = EngineConfig.defaults(str(model_dirs[name]), block_size=4, num_blocks=64)
    free = LLMEngine(cfg).generate([prompt], greedy(6))[0].token_ids
    e = LLMEngine(cfg, tokenizer=IntTokenizer())
    text_prompt = "".join(f"<{t}>" for t in prompt)
    out = e.generate([text_prompt], SamplingParams(max_tokens=6, stop=[f"<{free[2]}>"], ignore_eos=True))[0]
    cut = free.index(free[2])
    assert out.finish_reason == "stop" and out.text == "".join(f"<{t}>" for t in free[:cut])
    with pytest.raises(ValueError, match="tokenizer"):
        LLMEngine(cfg).add_request("t", prompt="<1><2>")
    with pytest.raises(ValueError, match="exactly one"):
        e.add_request("t")
    with pytest.raises(ValueError, match="outside the vocabulary"):
        e.add_request("t", prompt_token_ids=[999999])


def test_command_line(model_dirs, tmp_path, capsys):
    from clockwork_amd import cli

    name = "A"
    prompt = prompts_for(name, [7], seed=10)[0]
    yaml_path = tmp_path / "engine.yaml"
    yaml_path.write_text(f"model:\n  model: {model_dirs[name]}\ncache:\n  block_size: 4\n  num_blocks: 64\n")
    rc = cli.main(["--config", str(yaml_path), "--set", "dtype=float32", "--prompt-ids", ",".join(map(str, prompt)),
                   "--max-tokens", "5", "--ignore-eos"])
    assert rc == 0
    import json

    line = json.loads(capsys.readouterr().out.strip().splitlines()[-1])
    assert line["token_ids"] == PlainQwen2(model_dirs[name]).greedy(prompt, 5)
    with pytest.raises(SystemExit):
        cli.main(["--config", str(yaml_path), "--set", "nonsense=1", "--prompt-ids", "1"])


def test_command_line_with_random_weights_equals_the_written_folder(tmp_path, capsys):
    """``--model config.json --random-weights SEED`` serves the very model that ``make-random``
    writes into a folder from the same file and seed: the same tokens, and the plain
    implementation's on that folder."""
    import json

    from clockwork_amd import cli
    from tests.configs import TINY_B

    config_json = tmp_path / "tiny_b.json"
    config_json.write_text(json.dumps(TINY_B))
    common = ["--set", "block_size=8", "--set", "num_blocks=64", "--prompt-ids", "5,17,3", "--max-tokens", "8", "--ignore-eos"]
    assert cli.main(["--model", str(config_json), "--random-weights", "2", *common]) == 0
    from_seed = json.loads(capsys.readouterr().out.strip().splitlines()[-1])["token_ids"]
    folder = tmp_path / "written"
    assert cli.main(["make-random", "--config-json", str(config_json), "--seed", "2", "--out", str(folder)]) == 0
    capsys.readouterr()
    assert cli.main(["--model", str(folder), *common]) == 0
    from_folder = json.loads(capsys.readouterr().out.strip().splitlines()[-1])["token_ids"]
    assert from_seed == from_folder == PlainQwen2(folder).greedy([5, 17, 3], 8)
    # another seed is another model
    assert cli.main(["--model", str(config_json), "--random-weights", "3", *common]) == 0
    assert json.loads(capsys.readouterr().out.strip().splitlines()[-1])["token_ids"] != from_seed
    # and the configuration key does the same through the Python entry point
    from clockwork_amd.engine.llm_engine import LLMEngine

    cfg = EngineConfig.defaults(str(config_json), weights="random", weight_seed=2, block_size=8, num_blocks=64)
    assert LLMEngine(cfg).generate([[5, 17, 3]], greedy(8))[0].token_ids == from_seed


def test_cache_size_left_open_is_what_the_scheduler_can_use(model_dirs):
    # a tiny model on a large card: the cap (twice max_num_seqs requests of max_model_len tokens) decides
    eng = engine(model_dirs["A"], num_blocks=0, max_num_seqs=4, max_model_len=64)
    assert eng.runner.num_blocks == 2 * 4 * (64 // 4) == eng.manager.num_blocks
    prompts = prompts_for("A", [9, 17])
    plain = PlainQwen2(model_dirs["A"])
    for prompt, out in zip(prompts, eng.generate(prompts, greedy(6))):
        assert out.token_ids == plain.greedy(prompt, 6)


def test_abort_while_the_next_step_already_runs(model_dirs):
    """In a stretch of plain decoding the next step is put on the GPU before the current outputs
    are made. A request aborted at that moment loses the token that step makes for it; the others
    are untouched and every page comes back."""
    name = "B"
    prompts = prompts_for(name, [7, 12, 5], seed=9)
    eng = engine(model_dirs[name], enable_prefix_cache=False)
    for i, prompt in enumerate(prompts):
        eng.add_request(f"r{i}", prompt_token_ids=prompt, sampling_params=greedy(16))
    finals, aborted_after = {}, None
    while eng.has_unfinished_requests():
        for out in eng.step():
            assert out.request_id != "r1" or aborted_after is None, "an aborted request produced an output"
            if out.finished:
                finals[out.request_id] = out.token_ids
        if aborted_after is None and eng._started is not None:
            aborted_after = len(eng._seqs["r1"].output_token_ids)
            eng.abort_request("r1")
    assert aborted_after is not None and 0 < aborted_after < 16
    assert sorted(finals) == ["r0", "r2"]
    plain = PlainQwen2(model_dirs[name])
    assert finals["r0"] == plain.greedy(prompts[0], 16) and finals["r2"] == plain.greedy(prompts[2], 16)
    assert eng.manager.min_free_blocks() == eng.manager.num_blocks
    assert eng.stats()["lookahead_steps"] > 0


def test_sampled_tokens_do_not_depend_on_steps_queued_ahead(model_dirs):
    """Temperature sampling: a step queued before the tokens of the step before it have reached
    the host must make the same draws as one started afterwards (the n-th draw of a request is a
    function of its seed and n alone)."""
    from clockwork_amd.engine.llm_engine import LLMEngine

    name = "B"
    prompts = prompts_for(name, [9, 4, 30], seed=2)
    params = [SamplingParams(max_tokens=14, temperature=0.8, top_k=50, top_p=0.9, seed=100 + i, ignore_eos=True)
              for i in range(3)]

    def session(lookahead: bool):
        eng = LLMEngine(EngineConfig.defaults(str(model_dirs[name]), dtype="float32", block_size=4, num_blocks=128,
                                              watermark=0.0, lookahead=lookahead))
        for i, prompt in enumerate(prompts):
            eng.add_request(f"r{i}", prompt_token_ids=prompt, sampling_params=params[i])
        finals = {}
        while eng.has_unfinished_requests():
            for out in eng.step():
                if out.finished:
                    finals[out.request_id] = out.token_ids
        return finals, eng.stats()["lookahead_steps"]

    ahead, used = session(True)
    plain_order, unused = session(False)
    assert ahead == plain_order and used > 5 and unused == 0
    assert len({tuple(v) for v in ahead.values()}) == 3


# seeds 12 and 15 run out of pages for three requests at once while a step is decided ahead
@pytest.mark.parametrize("seed", [0, 1, 12, 15])
def test_long_random_session_equals_every_request_alone(model_dirs, seed):
    """Arrivals at random times, stop tokens, aborts, so few pages that requests are preempted,
    shared prefixes, steps queued ahead: every request that finishes gives the tokens and the
    reason it gives alone, and every page comes back."""
    import random

    name = "B"
    vocab = TINY_CONFIGS[name][0]["vocab_size"]
    rng = random.Random(seed)

    def make(num_blocks, max_seqs, prefix):
        return engine(model_dirs[name], block_size=8, num_blocks=num_blocks, watermark=0.01, max_num_seqs=max_seqs,
                      max_num_batched_tokens=96, max_model_len=400, enable_prefix_cache=prefix)

    shared = [rng.randrange(vocab) for _ in range(40)]
    requests = []
    for i in range(70):
        prompt = shared[: rng.choice([0, 16, 40])] + [rng.randrange(vocab) for _ in range(rng.choice([1, 3, 9, 30, 70, 150]))]
        stops = [rng.randrange(vocab) for _ in range(rng.choice([0, 0, 30, 120]))]
        requests.append((f"q{i}", prompt, rng.choice([2, 10, 40, 90]), stops))

    def params(n, stops):
        return SamplingParams(max_tokens=n, temperature=0.0, stop_token_ids=stops, ignore_eos=True)

    eng = make(num_blocks=140, max_seqs=12, prefix=True)
    finals, aborted, live = {}, set(), []
    arrivals = iter(requests)
    while True:
        for _ in range(rng.choice([0, 0, 1, 2])):
            r = next(arrivals, None)
            if r is not None:
                eng.add_request(r[0], prompt_token_ids=r[1], sampling_params=params(r[2], r[3]))
                live.append(r[0])
        if live and rng.random() < 0.03:
            victim = rng.choice(live)
            eng.abort_request(victim)
            aborted.add(victim)
            live.remove(victim)
        if not eng.has_unfinished_requests():
            if len(finals) + len(aborted) == len(requests):
                break
            continue
        for out in eng.step():
            assert out.request_id not in aborted
            if out.finished:
                finals[out.request_id] = (out.token_ids, out.finish_reason)
                live.remove(out.request_id)
    stats = eng.stats()
    assert stats["num_preempted_total"] > 0 and stats["lookahead_steps"] > 0 and stats["total_cached_tokens"] > 0
    assert any(reason == "stop" for _, reason in finals.values())
    eng.prefix_cache.reset()
    assert eng.manager.min_free_blocks() == eng.manager.num_blocks
    alone = make(num_blocks=200, max_seqs=2, prefix=False)
    for rid, prompt, n, stops in requests:
        if rid not in aborted:
            out = alone.generate([prompt], params(n, stops))[0]
            assert (out.token_ids, out.finish_reason) == finals[rid], rid
    # and the engine alone is right: a sample of the requests against the plain implementation
    plain = PlainQwen2(model_dirs[name])
    checked = 0
    for rid, prompt, n, stops in requests:
        if rid in aborted or n > 40 or checked == 12:
            continue
        want = []
        for token in plain.greedy(prompt, n):
            want.append(token)
            if token in stops:
                break
        assert finals[rid][0] == want, rid
        checked += 1
    assert checked == 12


@pytest.mark.parametrize("seed", range(12))
def test_random_engine_configurations_and_sessions(model_dirs, seed):
    """Engine options drawn at random (page size, pages, token budget, requests at a time, prefix
    cache, chunked prefill, looking ahead, watermark) and a session drawn at random (prompts of 1
    to 180 tokens that share openings of 0 to 64, greedy or seeded temperature / top-k / top-p
    sampling, stop tokens, 1 to 90 tokens, arrivals spread over the steps, a request aborted now
    and then), in float32: every request that finishes gives the tokens and the reason it gives
    alone, an aborted one gives nothing more, and every page comes back."""
    import random

    from clockwork_amd.engine.llm_engine import LLMEngine

    rng = random.Random(seed)
    name = rng.choice(["A", "B", "C"])
    vocab = TINY_CONFIGS[name][0]["vocab_size"]
    block_size, budget = rng.choice([4, 8, 16]), rng.choice([16, 48, 96, 256])
    options = dict(dtype="float32", block_size=block_size, watermark=rng.choice([0.0, 0.02]), max_model_len=300,
                   max_num_seqs=rng.choice([2, 4, 12]), max_num_batched_tokens=budget,
                   enable_prefix_cache=rng.random() < 0.6, enable_chunked_prefill=rng.random() < 0.7,
                   lookahead=rng.random() < 0.7, seed=seed)
    if not options["enable_chunked_prefill"]:
        options["max_num_batched_tokens"] = max(budget, 200)  # every prompt fits a step whole
    opening = [rng.randrange(vocab) for _ in range(64)]
    requests = []
    for i in range(rng.randint(4, 30)):
        prompt = (opening[: rng.choice([0, 0, 8, 33, 64])] + [rng.randrange(vocab) for _ in range(rng.choice([1, 2, 9, 30, 70, 150]))])[:180]
        how = dict(temperature=0.0)
        if rng.random() < 0.5:
            how = dict(temperature=rng.choice([0.5, 1.0, 1.5]), top_k=rng.choice([-1, 1, 5, 50]), top_p=rng.choice([1.0, 0.9, 0.5]),
                       seed=rng.randrange(1000))
        stops = [rng.randrange(vocab) for _ in range(rng.choice([0, 0, 20]))]
        requests.append((f"q{i}", prompt, dict(max_tokens=rng.choice([1, 2, 10, 40, 90]), stop_token_ids=stops, ignore_eos=True, **how)))
    longest = max(len(prompt) + how["max_tokens"] for _, prompt, how in requests)
    num_blocks = max(-(-longest // block_size) + 2, rng.choice([20, 40, 100]))  # the longest request fits alone
    eng = LLMEngine(EngineConfig.defaults(str(model_dirs[name]), num_blocks=num_blocks, **options))
    finals, pending, live, aborted = {}, list(requests), set(), set()
    for _ in range(20000):
        if not pending and not eng.has_unfinished_requests():
            break
        for _ in range(rng.choice([0, 1, 1, 3])):
            if pending:
                rid, prompt, how = pending.pop(0)
                eng.add_request(rid, prompt_token_ids=prompt, sampling_params=SamplingParams(**how))
                live.add(rid)
        if live and rng.random() < 0.05:
            victim = rng.choice(sorted(live))
            eng.abort_request(victim)
            aborted.add(victim)
            live.discard(victim)
        if eng.has_unfinished_requests():
            for out in eng.step():
                assert out.request_id not in aborted
                if out.finished:
                    finals[out.request_id] = (out.token_ids, out.finish_reason)
                    live.discard(out.request_id)
    assert not pending and not eng.has_unfinished_requests() and len(finals) + len(aborted) == len(requests)
    eng.prefix_cache.reset()
    assert eng.manager.min_free_blocks() == eng.manager.num_blocks
    alone = LLMEngine(EngineConfig.defaults(str(model_dirs[name]), num_blocks=-(-longest // block_size) + 4,
                                            **dict(options, max_num_seqs=2, enable_prefix_cache=False, lookahead=False)))
    for rid, prompt, how in requests:
        if rid not in aborted:
            out = alone.generate([prompt], SamplingParams(**how))[0]
            assert (out.token_ids, out.finish_reason) == finals[rid], rid
