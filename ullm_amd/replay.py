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
    ap.add_argument("--enforce-eager", action="store_true", help="never replay decode steps from HIP graphs")
    return ap.parse_args(argv)


class Replayer:
    """The replay loop's state: the model, its runner and the live requests."""

    def __init__(self, model_dir: str, dtype: str, max_tokens: int, page_size: int = 16, device: str = "cuda:0",
                 max_requests: int = 8, use_graphs: bool = True):
        from .engine.loading import load_model
        from .engine.runner import ModelRunner
        if page_size < 1 or 64 % page_size:
            raise ValueError(f"page size {page_size} must divide 64")
        if max_tokens < 1:
            raise ValueError("max_tokens must be positive")
        self.max_tokens = -(-max_tokens // 64) * 64
        # max_tokens sizes the pool and bounds a request; a trace is replayed as given, also past the positions
        # the model's configuration names (that is said once, not refused)
        self.cfg, self.model, self.env = load_model(model_dir, dtype, device, context_len=self.max_tokens,
                                                    strict_context=False)
        self.runner = ModelRunner(self.model, self.env, page_size=page_size,
                                  num_pages=self.max_tokens // page_size, max_requests=max_requests,
                                  use_graphs=use_graphs)
        self.live = {}

    def step(self, msg: dict):
        """Run one step object; returns float32 logits [wanted, vocab] on the host or None."""
        from .engine.runner import StepEntry
        step = msg.get("step")
        entries = []
        for ent in msg.get("entries", []):
            rid = str(ent["id"])
            tokens = [int(t) for t in ent["tokens"]]
            if not tokens:
                continue
            rc = self.live.get(rid)
            if rc is None:
                rc = self.runner.cache.admit(rid)
                self.live[rid] = rc
            if not self.runner.cache.reserve(rc, len(tokens)):
                raise RuntimeError(
                    f"step {step}: request {rid!r} needs pages for {len(tokens)} more tokens but the pool made "
                    f"for {self.max_tokens} tokens has {self.runner.cache.num_free_pages()} pages left")
            entries.append(StepEntry(rc, tokens, [int(w) for w in ent.get("want", [])]))
        out = None
        if entries:
            logits = self.runner.step(entries)
            if logits is not None:
                out = logits.float().cpu().contiguous().numpy()
        for rid in msg.get("end", []):
            rc = self.live.pop(str(rid), None)
            if rc is not None:
                self.runner.cache.release(rc)
        return out


def main(argv=None) -> int:
    args = parse_args(argv)
    os.makedirs(args.out, exist_ok=True)
    try:
        rep = Replayer(args.model, args.dtype, args.max_tokens, args.page_size, args.device,
                       use_graphs=not args.enforce_eager)
    except ValueError as e:
        print(f"trace_run: {e}", file=sys.stderr)
        return 2
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        msg = json.loads(line)
        step = msg["step"]
        arr = rep.step(msg)
        if arr is not None:
            tmp = os.path.join(args.out, f".{step}.f32.tmp")
            arr.astype("<f4", copy=False).tofile(tmp)
            os.replace(tmp, os.path.join(args.out, f"{step}.f32"))
        sys.stdout.write(f"done {step}\n")
        sys.stdout.flush()
    return 0


if __name__ == "__main__":
    sys.exit(main())
