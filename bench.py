#!/usr/bin/env python3
"""Decode and prefill throughput of the engine at Qwen3 layer sizes with random weights.

    python bench.py --gpus 1 --steps K --warmup W

One JSON line.  ``value`` = decoded tokens per second at batch 8 of Qwen3-8B sizes (every request with a
1024-token prompt), timed over exactly K engine steps (schedule + model step + sampling) after W untimed
ones.  ``prefill`` = one 2048-token prompt.  ``roofline`` = bytes a decode step has to read (every weight
once + the live requests' cache) over its time, against 8 TB/s (``frac``) and against what a kernel that
only reads reaches on this GPU (``frac_of_measured``).  ``points`` = tokens per second of the other workloads
(decode at batch 1 and 64; batch 8 at 16K-token, batch 64 at 8K-token and batch 1 at 32K-token contexts; a
16,384-token prompt; Qwen3-14B and Qwen3-32B sizes at batch 8, Qwen3-32B at batch 64 with 4096-token contexts
and its 2048-token prefill; the 256-request mixed workloads at Qwen3-14B and Qwen3-0.6B sizes);
``points_detail`` says at which context each ran and how far from its roofline.  ``measured_peaks`` = a
streaming read, a device copy and a large bfloat16 product on this GPU.  The reference publishes no number for this configuration, so ``vs_baseline`` is null.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
PEAK_FLOPS = {"bfloat16": 2.5e15, "float32": 157.3e12}
# the reference's own benchmark (bench.py:10-45, README.md:129-147): Qwen3-0.6B, 256 requests, prompt and
# generation lengths uniform in 100..1024, temperature 0.6, no end-of-sequence; 9032.37 tokens/s on an A100 40GB
REFERENCE_MIXED_TOK_S = 9032.37
SIZES = ("0.6b", "8b", "14b", "32b")
LONGEST_CONTEXT = 32768 + 64       # the longest context any point of the default run reaches


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--layers", type=int, default=None, help="run fewer layers than the configuration has")
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--prompt-len", type=int, default=1024)
    ap.add_argument("--context-len", type=int, default=4096)
    ap.add_argument("--dtype", default="bfloat16")
    ap.add_argument("--top-k", type=int, default=-1, help="top-k of the decode requests (default: off)")
    ap.add_argument("--top-p", type=float, default=1.0, help="top-p of the decode requests (default: off)")
    ap.add_argument("--no-points", action="store_true", help="only the headline decode point")
    ap.add_argument("--eager", action="store_true", help="no HIP graphs")
    ap.add_argument("--size", choices=SIZES, default=None,
                    help="layer sizes of this Qwen3 model (default 8b; 0.6b for --mixed-only)")
    ap.add_argument("--mixed-only", action="store_true",
                    help="only the reference's own workload: 256 requests of mixed lengths "
                         "(Qwen3-0.6B sizes unless --size is given)")
    ap.add_argument("--prefill-only", type=int, default=0, metavar="T",
                    help="only time a T-token prompt and print its figures (for profiling)")
    return ap.parse_args()


def weight_bytes(model, itemsize):
    """Bytes of every weight a decode step reads once (the embedding table is only gathered)."""
    total = 0
    for d in model.weight_decls():
        if d.name == model.plan.embedding_weight and not model.plan.tie_head_to_embedding:
            continue
        n = 1
        for s in d.shape:
            n *= s
        total += n * (4 if d.keep_fp32 else itemsize)
    return total


def step_flops(cfg, n_tokens, kv_lens_sum_causal, n_logit_rows):
    """Multiply-adds * 2 of one step: projections per token, attention scores and values, head."""
    H, nq, nkv, hd, I, L, V = (cfg.hidden_size, cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim,
                               cfg.intermediate_size, cfg.num_hidden_layers, cfg.vocab_size)
    per_token = 2 * (H * (nq + 2 * nkv) * hd + nq * hd * H + 3 * H * I)
    attn = 4 * nq * hd * kv_lens_sum_causal
    return L * (per_token * n_tokens + attn) + 2 * H * V * n_logit_rows


def measured_peaks():
    """What this GPU reaches with a kernel that only reads (4 GiB, non-temporal 16-byte loads: what a decode
    step's weight streaming could reach at best), on a plain device-to-device copy (bytes read + written per
    second) and on a large square bfloat16 product of the library: the practical ceilings beside the datasheet's."""
    import torch
    from ullm_amd.kernels import ops
    src = torch.empty(1 << 30, dtype=torch.float32, device="cuda:0").normal_()
    for _ in range(2):
        ops.stream_read(src)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(5):
        ops.stream_read(src)
    torch.cuda.synchronize()
    read_gbs = 5 * src.numel() * 4 / (time.perf_counter() - t0) / 1e9
    dst = torch.empty_like(src)
    for _ in range(2):
        dst.copy_(src)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(5):
        dst.copy_(src)
    torch.cuda.synchronize()
    copy_gbs = 5 * 2 * src.numel() * 4 / (time.perf_counter() - t0) / 1e9
    del src, dst
    n = 8192
    a = torch.randn(n, n, device="cuda:0", dtype=torch.bfloat16)
    b = torch.randn(n, n, device="cuda:0", dtype=torch.bfloat16)
    for _ in range(3):
        torch.mm(a, b)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(10):
        torch.mm(a, b)
    torch.cuda.synchronize()
    gemm_tflops = 10 * 2 * n ** 3 / (time.perf_counter() - t0) / 1e12
    del a, b
    torch.cuda.empty_cache()
    return {"read_GBs": round(read_gbs, 1), "copy_GBs": round(copy_gbs, 1), "gemm_bf16_8192_TFLOPs": round(gemm_tflops, 1)}


class Sized:
    """A model of one named size with random weights on the device, and the runs it is timed on."""

    def __init__(self, size, dtype, context_len, layers=None, eager=False, longest_context=None):
        import torch
        from ullm_amd.config import parse_random_weights
        from ullm_amd.engine.loading import make_env
        from ullm_amd.models import build_model
        from ullm_amd.weights.random_init import bind_random_weights
        self.torch, self.size, self.dtype, self.context_len, self.eager = torch, size, dtype, context_len, eager
        config, _ = parse_random_weights(f"qwen3-{size}")
        self.full_layers = config["num_hidden_layers"]
        if layers is not None:
            config["num_hidden_layers"] = layers
        self.cfg, self.model = build_model(config)
        # the model (its position table) is built once for the longest context any point runs at; every engine
        # gets an environment with its own context length (block tables as wide as that context needs)
        self.env = make_env(dtype, "cuda:0", max(context_len, longest_context or 0))
        bind_random_weights(self.model, self.env, seed=0)
        self.itemsize = 2 if dtype == "bfloat16" else 4
        self.wbytes = weight_bytes(self.model, self.itemsize)
        self.kv_per_token = sum(g.bytes_per_token(self.itemsize) for g in self.model.cache_layout()[0])
        self.gen = torch.Generator().manual_seed(0)

    def engine(self, context_len=None, **kw):
        import dataclasses
        from ullm_amd import EngineConfig
        from ullm_amd.engine.engine import Engine
        context_len = context_len or self.context_len
        ec = EngineConfig(model="(random weights)", dtype=self.dtype, context_len=context_len, page_size=16,
                          enforce_eager=self.eager, **kw)
        return Engine(ec, model=self.model, env=dataclasses.replace(self.env, context_len=context_len), model_config=self.cfg)

    def _check_finite_once(self, eng):
        """The next step's logits must be finite (checked outside the timed steps)."""
        torch = self.torch

        def check(sampling, logits):
            eng.on_logits = None
            if not bool(torch.isfinite(logits).all()):
                raise RuntimeError(f"Qwen3-{self.size}: a step returned logits that are not finite")
        eng.on_logits = check

    def decode(self, batch, steps, warmup, prompt_len, top_k=-1, top_p=1.0, context_len=None):
        """(tokens/s, ms per step, bytes read per step, mean context) over exactly ``steps`` engine steps."""
        from ullm_amd import SamplingParams
        torch = self.torch
        budget = max(8192, batch)
        # requests that finish their prompt early decode while the others are still in theirs
        new_tokens = warmup + steps + 4 + -(-batch * prompt_len // budget)
        eng = self.engine(context_len=context_len, max_bs=batch, num_pages=batch * (-(-(prompt_len + new_tokens + 16) // 16)),
                          max_num_batched_tokens=budget, max_prefill_chunk=2048)
        for i in range(batch):
            prompt = torch.randint(0, self.cfg.vocab_size, (prompt_len,), generator=self.gen).tolist()
            eng.add_request(f"r{i}", prompt, SamplingParams(temperature=0.6, top_k=top_k, top_p=top_p, ignore_eos=True,
                                                            seed=i, max_new_tokens=new_tokens))
        while any(r.num_computed < prompt_len for r in eng.scheduler.requests.values()) or eng.scheduler.waiting:
            eng.step()                                   # prefill (untimed)
        self._check_finite_once(eng)
        for _ in range(max(1, warmup)):
            eng.step()
        ctx_before = sum(r.num_tokens for r in eng.scheduler.requests.values())
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            out = eng.step()
            assert len(out) == batch
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        ctx_after = sum(r.num_tokens for r in eng.scheduler.requests.values())
        mean_ctx = (ctx_before + ctx_after) / 2.0
        for rid in list(eng.scheduler.requests):
            eng.abort_request(rid)
        del eng
        torch.cuda.empty_cache()
        return batch * steps / dt, dt / steps * 1e3, self.wbytes + self.kv_per_token * mean_ctx, mean_ctx / batch

    def prefill(self, n_tokens):
        """(tokens/s, ms, fraction of the dtype's matrix peak) of one prompt of n_tokens, best of three."""
        from ullm_amd import SamplingParams
        torch = self.torch
        context_len = max(self.context_len, n_tokens + 16)
        if context_len > self.env.context_len:
            # the engine would keep the prompt's last context_len tokens and the figures would be of those
            raise SystemExit(f"a prompt of {n_tokens} tokens needs --context-len above {n_tokens} (it is {self.context_len})")
        eng = self.engine(context_len=context_len, max_bs=1, num_pages=-(-(n_tokens + 16) // 16),
                          max_num_batched_tokens=n_tokens, max_prefill_chunk=n_tokens)
        best = None
        for rep in range(4):
            prompt = torch.randint(0, self.cfg.vocab_size, (n_tokens,), generator=self.gen).tolist()
            eng.add_request(f"p{rep}", prompt, SamplingParams(temperature=0.0, max_new_tokens=1, ignore_eos=True))
            if rep == 0:
                self._check_finite_once(eng)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            out = eng.step()
            torch.cuda.synchronize()
            dt = time.perf_counter() - t0
            assert len(out) == 1 and out[0].is_finished
            if rep > 0:
                best = dt if best is None else min(best, dt)
        del eng
        torch.cuda.empty_cache()
        flops = step_flops(self.cfg, n_tokens, n_tokens * (n_tokens + 1) // 2, 1)
        return n_tokens / best, best * 1e3, flops / best / PEAK_FLOPS[self.dtype]

    def mixed(self):
        """Output tokens per second over 256 requests arriving at once (prompt and generation lengths uniform
        in 100..1024, temperature 0.6, no end-of-sequence), continuous batching; returns (tokens/s, output
        tokens, seconds, engine steps)."""
        import random
        from ullm_amd import SamplingParams
        torch = self.torch
        rng = random.Random(0)
        n = 256
        prompts = [[rng.randint(0, 10000) for _ in range(rng.randint(100, 1024))] for _ in range(n)]
        new_tokens = [rng.randint(100, 1024) for _ in range(n)]
        eng = self.engine(max_bs=256, num_pages=n * 130, max_num_batched_tokens=8192, max_prefill_chunk=2048)
        eng.add_request("warm", prompts[0][:64], SamplingParams(temperature=0.6, ignore_eos=True, max_new_tokens=10))
        self._check_finite_once(eng)
        while eng.has_unfinished_requests():
            eng.step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(n):
            eng.add_request(f"m{i}", prompts[i], SamplingParams(temperature=0.6, ignore_eos=True, seed=i,
                                                                max_new_tokens=new_tokens[i]))
        steps = 0
        while eng.has_unfinished_requests():
            eng.step()
            steps += 1
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        del eng
        torch.cuda.empty_cache()
        return sum(new_tokens) / dt, sum(new_tokens), dt, steps

    def close(self):
        del self.model
        self.torch.cuda.empty_cache()


def decode_detail(tok_s, ms, bytes_step, ctx, read_gbs):
    achieved = bytes_step / (ms * 1e-3) / 1e9
    return {"tok_s": round(tok_s, 2), "ms_per_step": round(ms, 4), "context": round(ctx, 1),
            "GBs": round(achieved, 1), "frac": round(achieved / HBM_PEAK_GBS, 4),
            "frac_of_measured": round(achieved / read_gbs, 4) if read_gbs else None}


def main():
    args = parse_args()
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported")
        return 2
    if args.mixed_only:
        size = args.size or "0.6b"
        m = Sized(size, args.dtype, 4096, eager=args.eager)
        tok_s, n_out, secs, steps = m.mixed()
        print(json.dumps({"metric": f"output tok/s, 256 requests, lengths 100..1024 in and out, Qwen3-{size} sizes",
                          "value": round(tok_s, 1), "unit": "tokens/s", "output_tokens": n_out,
                          "seconds": round(secs, 3), "engine_steps": steps,
                          "vs_baseline": round(tok_s / REFERENCE_MIXED_TOK_S, 3) if size == "0.6b" else None,
                          "baseline": "9032.37 tokens/s, the reference with Qwen3-0.6B on an A100 40GB"}))
        return 0
    args.size = args.size or "8b"
    long_points = not args.no_points and not args.prefill_only
    m = Sized(args.size, args.dtype, args.context_len, args.layers, args.eager,
              longest_context=LONGEST_CONTEXT if long_points else args.prefill_only + 16)
    cfg = m.cfg
    if args.prefill_only:
        p_tok_s, p_ms, p_frac = m.prefill(args.prefill_only)
        print(json.dumps({"prefill": {"value": round(p_tok_s, 1), "tokens": args.prefill_only, "ms": round(p_ms, 3),
                                      "frac": round(p_frac, 4)}}))
        return 0
    peaks = measured_peaks() if not args.no_points else {}
    copy_gbs = peaks.get("read_GBs")        # the denominator of frac_of_measured: a kernel that only reads
    tok_s, ms, bytes_step, ctx = m.decode(args.batch, args.steps, args.warmup, args.prompt_len, args.top_k, args.top_p)
    head = decode_detail(tok_s, ms, bytes_step, ctx, copy_gbs)
    line = {
        "metric": f"decode tok/s at bs {args.batch} (also bs 1/64, prefill tok/s at 2048; % of roofline), Qwen3-{args.size}",
        "value": round(tok_s, 2), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32", "data": "synthetic",
        "config": {"model": f"Qwen3-{args.size} sizes, random weights", "layers": cfg.num_hidden_layers,
                   "layers_of_config": m.full_layers, "hidden_size": cfg.hidden_size,
                   "num_attention_heads": cfg.num_attention_heads, "num_key_value_heads": cfg.num_key_value_heads,
                   "head_dim": cfg.head_dim, "intermediate_size": cfg.intermediate_size, "vocab_size": cfg.vocab_size,
                   "global_batch": args.batch, "prompt_len": args.prompt_len, "seq_len": args.context_len,
                   "context_at_timing": head["context"], "page_size": 16,
                   "sampling": "temperature 0.6, seeded" + (f", top-k {args.top_k}" if args.top_k > 0 else "") + (f", top-p {args.top_p}" if args.top_p < 1 else ""),
                   "parallelism": "single GPU", "hip_graphs": not args.eager},
        "roofline": {"bound": "hbm", "achieved": head["GBs"], "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": head["frac"],
                     "frac_of_measured": head["frac_of_measured"]},
    }
    if not args.no_points:
        line["measured_peaks"] = peaks
        p_tok_s, p_ms, p_frac = m.prefill(2048)
        line["prefill"] = {"value": round(p_tok_s, 1), "tokens": 2048, "ms": round(p_ms, 3), "frac": round(p_frac, 4)}
        if peaks.get("gemm_bf16_8192_TFLOPs") and args.dtype == "bfloat16":
            line["prefill"]["frac_of_measured"] = round(p_frac * PEAK_FLOPS["bfloat16"] / (peaks["gemm_bf16_8192_TFLOPs"] * 1e12), 4)
        detail = {}
        b1 = m.decode(1, min(args.steps, 32), min(args.warmup, 4), args.prompt_len)
        b64 = m.decode(64, min(args.steps, 32), min(args.warmup, 4), args.prompt_len)
        # the same batch with the sampling of Qwen3's generation_config.json (top-k 20, top-p 0.95)
        b8f = m.decode(args.batch, args.steps, args.warmup, args.prompt_len, top_k=20, top_p=0.95)
        detail["decode_b1"] = decode_detail(*b1, copy_gbs)
        detail["decode_b64"] = decode_detail(*b64, copy_gbs)
        points = {"decode_b1": round(b1[0], 2), "decode_b64": round(b64[0], 2),
                  f"decode_b{args.batch}_top_k20_top_p95": round(b8f[0], 2)}
        if args.size == "8b" and args.dtype == "bfloat16":
            # further contexts: where the cache outweighs the weights
            for name, batch, ctx in (("decode_b8_ctx16k", 8, 16384), ("decode_b64_ctx8k", 64, 8192), ("decode_b1_ctx32k", 1, 32768)):
                d = m.decode(batch, 16, 2, ctx - 128, context_len=ctx + 64)
                detail[name] = decode_detail(*d, copy_gbs)
                points[name] = round(d[0], 2)
            p16 = m.prefill(16384)
            points["prefill_16384"] = round(p16[0], 1)
            detail["prefill_16384"] = {"tok_s": round(p16[0], 1), "ms": round(p16[1], 3), "frac": round(p16[2], 4)}
        m.close()
        if args.size == "8b" and args.layers is None and args.dtype == "bfloat16":
            # Qwen3-32B sizes: batch 64 with 4096-token contexts (about 69 GB of cache) and a 2048-token prompt
            big = Sized("32b", args.dtype, 4096 + 64, eager=args.eager)
            d32 = big.decode(64, 16, 2, 4096 - 32)
            detail["decode_32b_b64_ctx4096"] = decode_detail(*d32, copy_gbs)
            points["decode_32b_b64_ctx4096"] = round(d32[0], 2)
            d32 = big.decode(8, 16, 2, 1024)
            detail["decode_32b_b8"] = decode_detail(*d32, copy_gbs)
            points["decode_32b_b8"] = round(d32[0], 2)
            p32 = big.prefill(2048)
            points["prefill_32b_2048"] = round(p32[0], 1)
            detail["prefill_32b_2048"] = {"tok_s": round(p32[0], 1), "ms": round(p32[1], 3), "frac": round(p32[2], 4)}
            big.close()
            # the 256-request workload at Qwen3-14B sizes, and the reference's own at Qwen3-0.6B sizes
            mid = Sized("14b", args.dtype, 4096, eager=args.eager)
            d14 = mid.decode(8, 16, 2, 1024)
            detail["decode_14b_b8"] = decode_detail(*d14, copy_gbs)
            points["decode_14b_b8"] = round(d14[0], 2)
            m14 = mid.mixed()
            points["mixed_qwen3_14b"] = round(m14[0], 1)
            detail["mixed_qwen3_14b"] = {"output_tok_s": round(m14[0], 1), "output_tokens": m14[1],
                                         "seconds": round(m14[2], 3), "engine_steps": m14[3]}
            mid.close()
        small = Sized("0.6b", args.dtype, 4096, eager=args.eager)
        m_tok_s, m_out, m_secs, _ = small.mixed()
        small.close()
        points["mixed_qwen3_0p6b"] = round(m_tok_s, 1)
        line["points"] = points
        line["points_detail"] = detail
        # the reference's own benchmark (Qwen3-0.6B, 256 requests); its 9032.37 tokens/s are from an A100 40GB
        line["mixed_qwen3_0p6b"] = {"value": round(m_tok_s, 1), "unit": "output tokens/s", "output_tokens": m_out,
                                    "seconds": round(m_secs, 3),
                                    "vs_reference_a100": round(m_tok_s / REFERENCE_MIXED_TOK_S, 3)}
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
