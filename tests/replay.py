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


def run_trace(runner: ModelRunner, steps, usage: dict | None = None) -> dict:
    """``steps``: list of dicts {"entries": [{"id", "tokens", "want"}], "end": [...], and the
    optional "share" / "fork"} as trace_run reads them, run by the program's own ``TraceReplayer``.
    Returns {(id, absolute position): float32 logits row on the CPU}. ``usage`` (a dict) receives
    "peak_pages": the most pages of a pool that were held while a step ran."""
    from clockwork_amd.engine.trace_run import TraceReplayer

    replayer = TraceReplayer(runner)
    got = {}
    for step in steps:
        entries, logits = replayer.run_step(step)
        if logits is not None:
            logits = logits.cpu()
            row = 0
            for e in entries:
                for w in e.want:
                    got[(e.seq_id, e.start + w)] = logits[row]
                    row += 1
            assert row == logits.shape[0]
    if usage is not None:
        usage["peak_pages"] = replayer.peak_pages
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


def shared(a: list, vocab: int, block_size: int, seed: int = 0):
    """Requests that hold the same pages. ``a`` is the tokens of request A, which runs throughout;
    beside it, at most four live at a time:

    * C is forked from A in the middle of a page; in that step A writes first, so A gets the copy;
    * B begins with A's first two pages (a prefix-cache hit: the share ends at a page's edge);
    * D begins with A's first page and three tokens of the second: it writes into a page that
      A, B and C hold as well, behind tokens of A's that are not D's;
    * G is forked from A later and writes first, so the child gets the copy;
    * E and F are strangers that arrive when others have ended and take the pages given back,
      among them pages that were copied from and copied to.

    Every request goes on with tokens of its own, in portions and single tokens, and every
    position's logits are wanted. Returns (steps, {id: the request's whole token sequence},
    {id: the position at which the request's own steps begin})."""
    import random

    rng = random.Random(seed)
    bs = block_size
    fork_at = 2 * bs + bs // 2 + 1
    assert len(a) >= fork_at + 3 * bs, "request A is too short for this trace"

    def tail(n):
        return [rng.randrange(vocab) for _ in range(n)]

    seqs = {"A": list(a)}
    at: dict[str, int] = {}
    starts: dict[str, int] = {"A": 0}
    live: list[str] = []
    steps: list[dict] = []
    sizes = [3, 1, 1, 5, 1, 2, 1, 1, 7, 1]

    def join(step, rid, kind, count=None, own=0):
        if kind == "fork":
            seqs[rid] = seqs["A"][: at["A"]] + tail(own)
            at[rid] = at["A"]
            step.setdefault("fork", []).append({"id": rid, "from": "A"})
        elif kind == "share":
            seqs[rid] = seqs["A"][:count] + tail(own)
            at[rid] = count
            step.setdefault("share", []).append({"id": rid, "from": "A", "tokens": count})
        else:
            seqs[rid] = tail(own)
            at[rid] = 0
        starts[rid] = at[rid]
        live.append(rid)

    # who joins, as soon as fewer than four requests are live (A must still be there for a fork)
    arrivals = [("C", "fork", None, 2 * bs + 3), ("B", "share", 2 * bs, bs + 5), ("D", "share", bs + 3, 6),
                ("G", "fork", None, bs + 2), ("E", "new", None, 3 * bs + 1), ("F", "new", None, 2 * bs + 2)]
    at["A"] = 0
    live.append("A")
    steps.append({"entries": [{"id": "A", "tokens": a[:fork_at], "want": list(range(fork_at))}], "end": []})
    at["A"] = fork_at
    tick = 0
    while live:
        step: dict = {"entries": [], "end": []}
        joined = []
        while arrivals and len(live) < 4 and (arrivals[0][1] == "new" or "A" in live):
            rid, kind, count, own = arrivals.pop(0)
            join(step, rid, kind, count, own)
            joined.append(rid)
        if arrivals and "A" not in live and arrivals[0][1] != "new":
            raise AssertionError("request A ended before every fork and share was made")
        # A first in the step of C's fork (A copies), the newcomer first in G's (the child copies)
        order = list(live)
        if "G" in joined:
            order.remove("G")
            order.insert(0, "G")
        elif tick % 2 and not joined:
            order.reverse()
        for i, rid in enumerate(order):
            toks = seqs[rid]
            if rid == "A":
                n = 1
            elif rid in ("E", "F") and at[rid] == 0:
                n = len(toks) - 4
            else:
                n = sizes[(tick + i) % len(sizes)]
            n = min(n, len(toks) - at[rid])
            step["entries"].append({"id": rid, "tokens": toks[at[rid] : at[rid] + n], "want": list(range(n))})
            at[rid] += n
            if at[rid] == len(toks):
                step["end"].append(rid)
        assert len(live) <= 4
        live[:] = [rid for rid in live if rid not in step["end"]]
        steps.append(step)
        tick += 1
    assert not arrivals
    return steps, seqs, starts


def compare_to_scale(got: dict, plain_logits: dict, rms_bound: float = 2e-2, worst_bound: float = 1e-1) -> tuple:
    """For bfloat16, whose every activation is rounded to 8 bits: the errors relative to the
    logits' own scale (their root mean square over everything compared). Their root mean square
    must stay within ``rms_bound`` of it and the largest within ``worst_bound``: rounding gives
    about one hundredth, a wrong key, mask or weight row moves logits by the scale itself.
    Returns (scale, rms error, largest error)."""
    assert got, "the replay produced no logits"
    keys = sorted(got)
    ref = torch.stack([plain_logits[rid][pos] for rid, pos in keys]).float()
    rows = torch.stack([got[k] for k in keys])
    bad = torch.isnan(rows).any(dim=1)
    assert not bool(bad.any()), f"NaN in the logits of {keys[int(bad.nonzero()[0])]}"
    errors = rows - ref
    scale = ref.square().mean().sqrt().item()
    rms = errors.square().mean().sqrt().item()
    per_row = errors.abs().max(dim=1).values
    worst = per_row.max().item()
    assert rms < rms_bound * scale, f"rms error {rms:.3e} against a scale of {scale:.3e}"
    assert worst < worst_bound * scale, (
        f"request and position {keys[int(per_row.argmax())]}: error {worst:.3e} against a scale of {scale:.3e}")
    return scale, rms, worst


def sharpen(src_dir, dst_dir, score_std: float = 2.0):
    """A copy of a random-weights model folder whose attention is peaked: query and key
    projections scaled so that a score's standard deviation is about ``score_std`` instead of the
    few hundredths that N(0, 0.02) weights give. Then a few keys carry most of each softmax, and a
    key that is missed, read twice or read from a stale page moves the logits by their own scale
    (with near-uniform attention over a hundred keys it would move them by a hundredth of it).
    At 2.0 about one key in twenty of a hundred carries the softmax, and the rounding of bfloat16
    queries and keys, which the exponential magnifies, still stays inside the bfloat16 bound
    (measured: 1.2% root mean square, 8% at worst, of the logits' scale; 1.5% and 11% at 2.5)."""
    import json
    from pathlib import Path

    from safetensors.torch import load_file, save_file

    src_dir, dst_dir = Path(src_dir), Path(dst_dir)
    cfg = json.loads((src_dir / "config.json").read_text())
    # scores of unit-variance inputs through N(0, 0.02) projections: std = hidden * 0.02^2
    factor = (score_std / (cfg["hidden_size"] * 0.02 ** 2)) ** 0.5
    tensors = load_file(str(src_dir / "model.safetensors"))
    for name in list(tensors):
        if ".q_proj." in name or ".k_proj." in name:
            tensors[name] = (tensors[name].float() * factor).to(tensors[name].dtype)
    dst_dir.mkdir(parents=True, exist_ok=True)
    (dst_dir / "config.json").write_text(json.dumps(cfg))
    save_file(tensors, str(dst_dir / "model.safetensors"))
    return dst_dir


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


def random_trace(seed: int, vocab: int, kinds=("fork", "share")):
    """A random trace of three to six requests, at most four live at a time: portions of 2 to 200
    tokens and single tokens in any mix, requests left out of steps, wants at random places, and
    requests that begin as a fork of the request before them or with a share of its pages (cut at
    any token; ``kinds`` says which of the two a trace may hold). A request that another will derive
    from stays live until that one has begun. Returns (steps, {id: the request's whole token sequence})."""
    import random

    rng = random.Random(seed)
    seqs, derive = {}, {}
    for i in range(rng.randint(3, 6)):
        rid, prev = f"r{i}", f"r{i - 1}"
        if i and rng.random() < 0.5 and len(seqs[prev]) > 1:
            kind = rng.choice(list(kinds))
            # a fork is taken where the request before stands: not before that one's own beginning
            first = derive[prev][2] if kind == "fork" and prev in derive else 1
            cut = rng.randint(max(1, first), len(seqs[prev]) - 1)
            derive[rid] = (kind, prev, cut)
            seqs[rid] = seqs[prev][:cut] + [rng.randrange(vocab) for _ in range(rng.randint(2, 200))]
        else:
            seqs[rid] = [rng.randrange(vocab) for _ in range(rng.choice([1, 3, 20, 70, 150, 400]))]
    order = list(seqs)
    pos, live, steps, admitted = {}, [], [], 0
    while admitted < len(order) or live:
        step = {"entries": [], "end": [], "fork": [], "share": []}
        fresh = set()
        while admitted < len(order) and len(live) < 4:
            rid = order[admitted]
            if rid in derive:
                kind, src, cut = derive[rid]
                if pos[src] < cut or src in fresh:
                    break  # the request before has not come that far yet, or begins in this very step
                if kind == "fork":
                    assert pos[src] == cut, "the request before ran past the place of the fork"
                    step["fork"].append({"id": rid, "from": src})
                else:
                    step["share"].append({"id": rid, "from": src, "tokens": cut})
                pos[rid] = cut
            else:
                pos[rid] = 0
            live.append(rid)
            fresh.add(rid)
            admitted += 1
        busy = [r for r in live if pos[r] < len(seqs[r])]
        for rid in list(live):
            left = len(seqs[rid]) - pos[rid]
            index = order.index(rid)
            heir = order[index + 1] if index + 1 < len(order) and index + 1 >= admitted else None
            heir = heir if heir in derive and derive[heir][1] == rid else None
            waits = heir is not None and derive[heir][0] == "fork" and pos[rid] == derive[heir][2]  # for the fork to be taken
            if left and not waits and not (len(busy) > 1 and rng.random() < 0.15):
                n = 1 if rng.random() < 0.5 else rng.choice([2, 3, 7, 16, 33, 64, 100, 200])
                if heir and derive[heir][0] == "fork" and pos[rid] < derive[heir][2]:
                    n = min(n, derive[heir][2] - pos[rid])  # stop where the fork will be taken
                n = max(1, min(n, left))
                want = sorted(rng.sample(range(n), rng.randint(0, min(n, 3))))
                step["entries"].append({"id": rid, "tokens": seqs[rid][pos[rid] : pos[rid] + n], "want": want})
                pos[rid] += n
            if pos[rid] == len(seqs[rid]) and heir is None:
                step["end"].append(rid)
                live.remove(rid)
        if step["entries"] or step["end"] or step["fork"] or step["share"]:
            steps.append(step)
    return steps, seqs
