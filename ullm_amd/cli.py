"""Offline generator: ``python -m ullm_amd.cli --model DIR --prompt-ids 1,2,3``.

Engine options carry the reference's names and defaults (ullm/entrypoints/api_server.py:126-183,
the reference's only command line, which starts its server); the generation options are the fields
of ``SamplingParams``.
"""
from __future__ import annotations

import argparse
import json
import sys

from .config.engine_config import EngineConfig
from .sampling import SamplingParams


def build_parser() -> argparse.ArgumentParser:
    ap = argparse.ArgumentParser(prog="ullm_amd", description="Generate with a Qwen3 model folder on one MI355X")
    EngineConfig.add_cli_args(ap)
    src = ap.add_argument_group("prompts (token ids are the primary interface)")
    src.add_argument("--prompt-ids", action="append", default=[],
                     help="comma-separated token ids; may be given several times")
    src.add_argument("--prompt", action="append", default=[], help="text prompt (needs the model's tokenizer)")
    src.add_argument("--prompts-file", type=str, default=None,
                     help="JSON lines: a list of token ids or a string per line")
    gen = ap.add_argument_group("sampling")
    gen.add_argument("--temperature", type=float, default=None, help="0 = greedy")
    gen.add_argument("--top-k", type=int, default=None)
    gen.add_argument("--top-p", type=float, default=None)
    gen.add_argument("--min-p", type=float, default=None)
    gen.add_argument("--max-tokens", type=int, default=None, help="cap on prompt + generated tokens")
    gen.add_argument("--max-new-tokens", type=int, default=16, help="cap on generated tokens")
    gen.add_argument("--ignore-eos", action="store_true")
    gen.add_argument("--request-seed", type=int, default=None, help="seed of every request (default: engine seed + order)")
    return ap


def main(argv=None) -> int:
    args = build_parser().parse_args(argv)
    prompts = [[int(x) for x in s.split(",") if x.strip()] for s in args.prompt_ids] + list(args.prompt)
    if args.prompts_file:
        with open(args.prompts_file) as f:
            prompts += [json.loads(line) for line in f if line.strip()]
    if not prompts:
        print("no prompt given: use --prompt-ids, --prompt or --prompts-file", file=sys.stderr)
        return 2
    from .llm import LLM
    config = EngineConfig.from_args(args)
    llm = LLM(config)
    base = config.generation_defaults()
    for key in ("temperature", "top_k", "top_p", "min_p"):
        if getattr(args, key) is not None:
            base[key] = getattr(args, key)
    params = [SamplingParams(max_tokens=args.max_tokens, max_new_tokens=args.max_new_tokens,
                             ignore_eos=args.ignore_eos, seed=args.request_seed, **base) for _ in prompts]
    for out in llm.generate(prompts, params):
        print(json.dumps({"prompt_tokens": out.num_prompt_tokens, "token_ids": out.token_ids, "text": out.text,
                          "finish_reason": out.finish_reason.name if out.finish_reason else None}))
    llm.shutdown()
    return 0


if __name__ == "__main__":
    sys.exit(main())
