r"""Command line: offline generation from a config file plus KEY=VALUE overrides.

The option style is the reference's launcher (scripts/serve.py:33-55: ``--config`` naming a
YAML file with ``model:``, ``cache:``, ``scheduler:`` sections, repeatable ``--set KEY=VALUE``
with the value read as YAML and routed to every section that has the key). Instead of
starting a server it generates for the prompts given and prints one JSON line per request.

    python -m clockwork_amd.cli --config engine.yaml --set dtype=bfloat16 \
        --prompt-ids 5,17,3 --prompt-ids 9,9,9 --max-tokens 16 --temperature 0.8 --seed 1

    python -m clockwork_amd.cli --model config.json --random-weights 2 --prompt-ids 5,17,3 --max-tokens 8

    python -m clockwork_amd.cli make-random --config-json config.json --seed 0 --out DIR
"""

from __future__ import annotations

import argparse
import json
import sys

from clockwork_amd.config.engine import EngineConfig
from clockwork_amd.engine.sequence import SamplingParams


def parse_generate(argv):
    """(arguments, engine configuration, prompts) of a generation command line; touches no GPU."""
    p = argparse.ArgumentParser(prog="clockwork-generate", description=__doc__,
                                formatter_class=argparse.RawDescriptionHelpFormatter)
    p.add_argument("--config", help="engine YAML (sections model / cache / scheduler)")
    p.add_argument("--model", help="model folder; stands in for --config with defaults")
    p.add_argument("--random-weights", type=int, default=None, metavar="SEED",
                   help="serve random weights drawn from SEED instead of a checkpoint (the values that "
                        "make-random writes); --model may then name a bare config.json")
    p.add_argument("--set", dest="overrides", action="append", default=[], metavar="KEY=VALUE",
                   help="override any model, cache or scheduler field, e.g. --set num_blocks=1024")
    p.add_argument("--prompt-ids", action="append", default=[], metavar="I,J,K", help="a prompt as token ids")
    p.add_argument("--prompt-file", help="file with one JSON list of token ids per line")
    p.add_argument("--prompt", action="append", default=[], help="a text prompt (needs --tokenizer)")
    p.add_argument("--tokenizer", help="folder of a tokenizers/transformers tokenizer, for text in and out")
    p.add_argument("--max-tokens", type=int, default=64)
    p.add_argument("--temperature", type=float, default=0.0)
    p.add_argument("--top-p", type=float, default=1.0)
    p.add_argument("--top-k", type=int, default=-1)
    p.add_argument("--seed", type=int, default=None)
    p.add_argument("--ignore-eos", action="store_true")
    p.add_argument("--stop-token-ids", default="", metavar="I,J")
    p.add_argument("--stop", action="append", default=[], metavar="TEXT", help="a stop string (needs --tokenizer)")
    args = p.parse_args(argv)

    if (args.config is None) == (args.model is None):
        p.error("give exactly one of --config and --model")
    cfg = EngineConfig.from_yaml(args.config) if args.config else EngineConfig.defaults(args.model)
    try:
        if args.random_weights is not None:
            cfg.set("weights", "random")
            cfg.set("weight_seed", args.random_weights)
        cfg.apply_overrides(args.overrides)
    except ValueError as e:
        raise SystemExit(str(e))

    prompts: list = [[int(t) for t in s.split(",") if t.strip()] for s in args.prompt_ids]
    if args.prompt_file:
        with open(args.prompt_file, encoding="utf-8") as f:
            prompts += [json.loads(line) for line in f if line.strip()]
    prompts += args.prompt
    if not prompts:
        p.error("no prompts: use --prompt-ids, --prompt-file or --prompt")
    return args, cfg, prompts


def _generate(argv) -> int:
    args, cfg, prompts = parse_generate(argv)
    tokenizer = None
    if args.tokenizer:
        from transformers import AutoTokenizer  # tokenizer files only; no model code is involved

        tokenizer = AutoTokenizer.from_pretrained(args.tokenizer)

    from clockwork_amd.engine.llm_engine import LLMEngine

    engine = LLMEngine(cfg, tokenizer=tokenizer)
    params = SamplingParams(
        max_tokens=args.max_tokens, temperature=args.temperature, top_p=args.top_p, top_k=args.top_k,
        seed=args.seed, ignore_eos=args.ignore_eos,
        stop_token_ids=[int(t) for t in args.stop_token_ids.split(",") if t.strip()], stop=list(args.stop),
    )
    for out in engine.generate(prompts, params):
        print(json.dumps({
            "request_id": out.request_id,
            "prompt_token_ids": out.prompt_token_ids,
            "token_ids": out.token_ids,
            "text": out.text,
            "finish_reason": out.finish_reason,
            "num_cached_tokens": out.num_cached_tokens,
        }))
    print(json.dumps({"stats": engine.stats()}), file=sys.stderr)
    return 0


def _make_random(argv) -> int:
    p = argparse.ArgumentParser(prog="clockwork-generate make-random",
                                description="write config.json and model.safetensors with random weights")
    p.add_argument("--config-json", required=True, help="a config.json of a supported architecture")
    p.add_argument("--seed", type=int, default=0)
    p.add_argument("--out", required=True)
    p.add_argument("--dtype", choices=("bfloat16", "float32"), default="bfloat16",
                   help="how the tensors are stored; float32 keeps the full mantissas of the drawn values")
    args = p.parse_args(argv)
    from clockwork_amd.weights.random_init import write_random_model

    with open(args.config_json, encoding="utf-8") as f:
        config = json.load(f)
    print(write_random_model(args.out, config, args.seed, dtype=args.dtype))
    return 0


def main(argv=None) -> int:
    argv = list(sys.argv[1:] if argv is None else argv)
    if argv and argv[0] == "make-random":
        return _make_random(argv[1:])
    return _generate(argv)


if __name__ == "__main__":
    sys.exit(main())
