"""Trace replay: feed given token ids through the model step by step and write logits.

It samples nothing and owns no forward pass, cache or loader: it drives the same model, step
function, cache manager and kernels that generation uses.  Steps arrive on standard input, one
JSON object a line:

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

For a step in which something is wanted, ``<out>/<step>.f32`` receives the logits at the wanted
places (order of the entries, then of ``want``) as little-endian float32 [wanted, vocab].  After
every step a line ``done <step>`` is printed and flushed.
"""
from __future__ import annotations

import argparse
import json
import os
import sys

import numpy as np


def parse_args(argv=None):
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True, help="folder for <step>.f32 files")
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="most tokens live requests hold at any time (each rounded up to 64)")
    ap.add_argument("--page-size", type=int, default=16, help="tokens per cache page (divides 64)")
    ap.add_argument("--device", default="cuda:0")
    return ap.parse_args(argv)


def main(argv=None) -> int:
    args = parse_args(argv)
    if args.page_size < 1 or 64 % args.page_size:
        print(f"trace_run: --page-size {args.page_size} must divide 64", file=sys.stderr)
        return 2
    if args.max_tokens < 1:
        print("trace_run: --max-tokens must be positive", file=sys.stderr)
        return 2
    os.makedirs(args.out, exist_ok=True)

    import torch
    from .engine.loading import load_model
    from .engine.runner import ModelRunner, StepEntry

    max_tokens = -(-args.max_tokens // 64) * 64
    num_pages = max_tokens // args.page_size
    cfg, model, env = load_model(args.model, args.dtype, args.device, context_len=max_tokens)
    runner = ModelRunner(model, env, page_size=args.page_size, num_pages=num_pages, max_requests=8)
    live = {}

    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        msg = json.loads(line)
        step = msg["step"]
        entries = []
        for ent in msg.get("entries", []):
            rid = str(ent["id"])
            tokens = [int(t) for t in ent["tokens"]]
            if not tokens:
                continue
            rc = live.get(rid)
            if rc is None:
                rc = runner.cache.admit(rid)
                live[rid] = rc
            if not runner.cache.reserve(rc, len(tokens)):
                raise RuntimeError(
                    f"step {step}: request {rid!r} needs pages for {len(tokens)} more tokens but the pool made "
                    f"for --max-tokens {args.max_tokens} has {runner.cache.num_free_pages()} pages left")
            entries.append(StepEntry(rc, tokens, [int(w) for w in ent.get("want", [])]))
        if entries:
            logits = runner.step(entries)
            if logits is not None:
                arr = logits.to("cpu", torch.float32).contiguous().numpy().astype("<f4", copy=False)
                tmp = os.path.join(args.out, f".{step}.f32.tmp")
                arr.tofile(tmp)
                os.replace(tmp, os.path.join(args.out, f"{step}.f32"))
        for rid in msg.get("end", []):
            rc = live.pop(str(rid), None)
            if rc is not None:
                runner.cache.release(rc)
        sys.stdout.write(f"done {step}\n")
        sys.stdout.flush()
    return 0


if __name__ == "__main__":
    sys.exit(main())
