"""Trace replay: feed given token ids through the model step by step and write logits.

    trace_run --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N

Reads one JSON object a line from standard input,
``{"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}``,
runs each step's entries as one batch through the engine's own step function, cache
manager and kernels, and writes ``<out>/<step>.f32`` (little-endian float32
[wanted, vocab]) when something is wanted. After every step it prints ``done <step>``.
It samples nothing and schedules nothing.
"""

from __future__ import annotations

import argparse
import json
import sys
from pathlib import Path

PAGE = 16


def main(argv=None) -> int:
    parser = argparse.ArgumentParser(prog="trace_run", description=__doc__)
    parser.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    parser.add_argument("--dtype", choices=("bfloat16", "float32"), default="bfloat16")
    parser.add_argument("--out", required=True, help="folder the logits files go to")
    parser.add_argument("--max-tokens", type=int, required=True,
                        help="most tokens live requests hold at a time (each rounded up to 64)")
    args = parser.parse_args(argv)

    from clockwork_amd.config.engine import EngineConfig
    from clockwork_amd.engine.batch import StepEntry
    from clockwork_amd.engine.model_runner import ModelRunner

    out_dir = Path(args.out)
    out_dir.mkdir(parents=True, exist_ok=True)
    cfg = EngineConfig.defaults(
        args.model,
        dtype=args.dtype,
        block_size=PAGE,
        num_blocks=max(1, -(-args.max_tokens // PAGE)),
        # one request may hold every token of the pool
        max_model_len=max(PAGE, PAGE * -(-args.max_tokens // PAGE)),
        enable_prefix_cache=False,
        watermark=0.0,
    )
    runner = ModelRunner(cfg)
    lengths: dict[str, int] = {}
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        obj = json.loads(line)
        step = obj["step"]
        entries = []
        for e in obj.get("entries", []):
            seq_id = str(e["id"])
            tokens = [int(t) for t in e["tokens"]]
            start = lengths.get(seq_id, 0)
            runner.reserve(seq_id, start, len(tokens))
            entries.append(StepEntry(seq_id, start, tokens, [int(w) for w in e.get("want", [])]))
            lengths[seq_id] = start + len(tokens)
        logits = runner.step(entries)
        if logits is not None:
            logits.cpu().numpy().astype("<f4").tofile(out_dir / f"{step}.f32")
        for seq_id in obj.get("end", []):
            runner.release(str(seq_id))
            lengths.pop(str(seq_id), None)
        print(f"done {step}", flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
