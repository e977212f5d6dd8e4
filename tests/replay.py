"""Helpers that replay token traces through the engine's step function and compare with the
plain implementation."""

from __future__ import annotations

import torch

from clockwork_amd.config.engine import EngineConfig
from clockwork_amd.engine.batch import StepEntry
from clockwork_amd.engine.model_runner import ModelRunner


def make_runner(model_dir, dtype: str, block_size: int, num_blocks: int, poison: float = float("nan"),
                use_graphs: bool = True, max_model_len: int = 512) -> ModelRunner:
    cfg = EngineConfig.defaults(
        str(model_dir), dtype=dtype, block_size=block_size, num_blocks=num_blocks,
        enable_prefix_cache=False, watermark=0.0, max_model_len=max_model_len,
    )
    return ModelRunner(cfg, cache_fill=poison, use_graphs=use_graphs)


def run_trace(runner: ModelRunner, steps) -> dict:
    """``steps``: list of dicts {"entries": [{"id", "tokens", "want"}], "end": [...]} as trace_run
    reads them. Returns {(id, absolute position): float32 logits row on the CPU}."""
    lengths: dict[str, int] = {}
    got = {}
    for step in steps:
        entries = []
        for e in step["entries"]:
            start = lengths.get(e["id"], 0)
            runner.reserve(e["id"], start, len(e["tokens"]))
            entries.append(StepEntry(e["id"], start, e["tokens"], e.get("want", [])))
            lengths[e["id"]] = start + len(e["tokens"])
        logits = runner.step(entries)
        if logits is not None:
            logits = logits.cpu()
            row = 0
            for e in entries:
                for w in e.want:
                    got[(e.seq_id, e.start + w)] = logits[row]
                    row += 1
            assert row == logits.shape[0]
        for seq_id in step.get("end", []):
            runner.release(seq_id)
            lengths.pop(seq_id, None)
    return got


def whole(requests: dict) -> list:
    """Each request alone and whole: one step per request, every position wanted."""
    return [
        {"entries": [{"id": rid, "tokens": toks, "want": list(range(len(toks)))}], "end": [rid]}
        for rid, toks in requests.items()
    ]


def prefill_then_decode(requests: dict, tail: int = 32) -> list:
    """Most of a request in one step, its last ``tail`` tokens one by one."""
    steps = []
    for rid, toks in requests.items():
        head = max(1, len(toks) - tail)
        steps.append({"entries": [{"id": rid, "tokens": toks[:head], "want": list(range(head))}], "end": []})
        for p in range(head, len(toks)):
            steps.append({"entries": [{"id": rid, "tokens": toks[p : p + 1], "want": [0]}], "end": []})
        steps[-1]["end"] = [rid]
    return steps


PORTIONS = [2, 7, 3, 16, 5, 2, 31, 9, 64, 2, 17, 33]


def portions(requests: dict, sizes=PORTIONS) -> list:
    """Each request in portions of changing size, down to two tokens."""
    steps = []
    for rid, toks in requests.items():
        at, i = 0, 0
        while at < len(toks):
            n = min(sizes[i % len(sizes)], len(toks) - at)
            steps.append({"entries": [{"id": rid, "tokens": toks[at : at + n], "want": list(range(n))}], "end": []})
            at += n
            i += 1
        steps[-1]["end"] = [rid]
    return steps


def mixed(requests: dict, live: int = 4, decode_tail: int = 8, sizes=PORTIONS) -> list:
    """Up to ``live`` requests at a time: portions of some beside single tokens of others;
    a request that ends makes room (and pages) for the next."""
    waiting = list(requests.items())
    active: list[list] = []  # [id, tokens, position, portion counter]
    steps = []
    tick = 0
    while waiting or active:
        while waiting and len(active) < live:
            rid, toks = waiting.pop(0)
            active.append([rid, toks, 0, len(active) + tick])
        entries, ended = [], []
        for slot, rec in enumerate(active):
            rid, toks, at, i = rec
            if (tick + slot) % 5 == 4 and len(active) > 1:
                continue  # a request may be left out of a step and go on later
            if at < len(toks) - decode_tail:
                n = min(sizes[i % len(sizes)], len(toks) - decode_tail - at)
            else:
                n = 1
            entries.append({"id": rid, "tokens": toks[at : at + n], "want": list(range(n))})
            rec[2] = at + n
            rec[3] = i + 1
            if rec[2] == len(toks):
                ended.append(rid)
        if entries:
            steps.append({"entries": entries, "end": ended})
        active = [rec for rec in active if rec[0] not in ended]
        tick += 1
    return steps


def pages_needed(requests: dict, live: int, block_size: int) -> int:
    longest = sorted((len(t) for t in requests.values()), reverse=True)[:live]
    return sum(-(-n // block_size) for n in longest)


def compare(got: dict, plain_logits: dict, rtol: float, atol: float) -> float:
    """Every produced row against the plain implementation; returns the largest absolute error."""
    worst = 0.0
    assert got, "the replay produced no logits"
    for (rid, pos), row in sorted(got.items()):
        ref = plain_logits[rid][pos]
        assert not torch.isnan(row).any(), f"request {rid} position {pos}: NaN in the logits"
        err = (row - ref).abs()
        bound = atol + rtol * ref.abs()
        if bool((err > bound).any()):
            j = int((err - bound).argmax())
            raise AssertionError(
                f"request {rid}, position {pos}: logit {j} is {float(row[j])}, plain {float(ref[j])} "
                f"(error {float(err[j]):.3e}, allowed {float(bound[j]):.3e})"
            )
        worst = max(worst, float(err.max()))
    return worst
