"""Trace replay: feed given token ids through the model step by step and write logits.

    trace_run --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N [--page TOKENS]

Reads one JSON object a line from standard input,
``{"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}``,
runs each step's entries as one batch through the engine's own step function, cache
manager and kernels, and writes ``<out>/<step>.f32`` (little-endian float32
[wanted, vocab]) when something is wanted. After every step it prints ``done <step>``.
It samples nothing and schedules nothing.

Two optional fields of a step make requests that share pages, before the step's entries run:

* ``"share": [{"id": "b", "from": "a", "tokens": 32}]``: a new request ``b`` begins with the
  first 32 tokens that the live request ``a`` has cached (what a prefix-cache hit does): it
  holds ``a``'s pages for them and goes on at position 32 with tokens of its own. The count
  need not end at a page's edge: a page that both hold is copied for whoever writes to it first.
* ``"fork": [{"id": "c", "from": "a"}]``: ``c`` shares everything ``a`` has cached so far
  (pages shared, fixed-size state copied) and goes on from ``a``'s length.
"""

from __future__ import annotations

import argparse
import json
import sys
from pathlib import Path
from typing import Optional

PAGE = 16


class TraceReplayer:
    """Runs trace steps (dicts as the program reads them) on a ``ModelRunner``: takes pages,
    shares and forks, calls the step function, gives pages back. Keeps each live request's length."""

    def __init__(self, runner) -> None:
        self.runner = runner
        self.lengths: dict[str, int] = {}
        self.peak_pages = 0  # the most pages of one pool that were held while a step ran

    def _new_id(self, obj, key: str) -> str:
        seq_id = str(obj[key])
        if seq_id in self.lengths:
            raise ValueError(f"request {seq_id} is live already")
        return seq_id

    def run_step(self, obj: dict):
        """One step; returns ``(entries, logits)``: the step's ``StepEntry`` list and float32
        logits [wanted, vocab] on the device, or None when nothing was wanted."""
        from clockwork_amd.engine.batch import StepEntry

        for share in obj.get("share", []):
            seq_id, source = self._new_id(share, "id"), str(share["from"])
            have = self.lengths.get(source)
            if have is None:
                raise ValueError(f"request {source}, to share with {seq_id}, is not live")
            count = int(share.get("tokens", have))
            if not 0 < count <= have:
                raise ValueError(f"request {source} has {have} tokens cached, {count} cannot be shared")
            self.runner.share_prefix(seq_id, source, count)
            self.lengths[seq_id] = count
        for fork in obj.get("fork", []):
            seq_id, source = self._new_id(fork, "id"), str(fork["from"])
            if source not in self.lengths:
                raise ValueError(f"request {source}, to fork {seq_id} from, is not live")
            self.runner.fork(source, seq_id)
            self.lengths[seq_id] = self.lengths[source]
        entries = []
        for e in obj.get("entries", []):
            seq_id = str(e["id"])
            tokens = [int(t) for t in e["tokens"]]
            start = self.lengths.get(seq_id, 0)
            self.runner.reserve(seq_id, start, len(tokens))
            entries.append(StepEntry(seq_id, start, tokens, [int(w) for w in e.get("want", [])]))
            self.lengths[seq_id] = start + len(tokens)
        manager = self.runner.manager
        self.peak_pages = max(self.peak_pages, manager.num_blocks - manager.min_free_blocks())
        logits = self.runner.step(entries)
        for seq_id in obj.get("end", []):
            self.runner.release(str(seq_id))
            self.lengths.pop(str(seq_id), None)
        return entries, logits


def replay_config(model: str, dtype: str, max_tokens: int, page: int = PAGE):
    """The engine configuration of a replay: a pool of just the pages that ``max_tokens`` tokens
    need (each live request's count rounded up to pages), so that pages are used again; one
    request may hold them all; nothing is kept for later requests."""
    from clockwork_amd.config.engine import EngineConfig

    pages = max(1, -(-max_tokens // page))
    return EngineConfig.defaults(
        model, dtype=dtype, block_size=page, num_blocks=pages, max_model_len=page * pages,
        enable_prefix_cache=False, watermark=0.0,
    )


def main(argv: Optional[list] = None) -> int:
    parser = argparse.ArgumentParser(prog="trace_run", description=__doc__,
                                     formatter_class=argparse.RawDescriptionHelpFormatter)
    parser.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    parser.add_argument("--dtype", choices=("bfloat16", "float32"), default="bfloat16")
    parser.add_argument("--out", required=True, help="folder the logits files go to")
    parser.add_argument("--max-tokens", type=int, required=True,
                        help="most tokens live requests hold at a time (each rounded up to 64)")
    parser.add_argument("--page", type=int, default=PAGE, metavar="TOKENS",
                        help=f"tokens a page of the cache holds (default {PAGE})")
    args = parser.parse_args(argv)
    if args.page < 1:
        parser.error("--page must be at least 1")

    from clockwork_amd.engine.model_runner import ModelRunner

    out_dir = Path(args.out)
    out_dir.mkdir(parents=True, exist_ok=True)
    replayer = TraceReplayer(ModelRunner(replay_config(args.model, args.dtype, args.max_tokens, args.page)))
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        obj = json.loads(line)
        step = obj["step"]
        _, logits = replayer.run_step(obj)
        if logits is not None:
            logits.cpu().numpy().astype("<f4").tofile(out_dir / f"{step}.f32")
        print(f"done {step}", flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
