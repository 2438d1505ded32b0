#!/usr/bin/env python3
"""Decode and prefill throughput of the engine at Qwen3-8B layer sizes with random weights.

    python bench.py --gpus 1 --steps K --warmup W

One JSON line: ``value`` = decoded tokens per second at batch 8 (every request with a 1024-token
prompt), timed over exactly K engine steps (schedule + model step + sampling) after W untimed ones;
``prefill`` = one 2048-token prompt; ``roofline`` = bytes a decode step has to read (every weight
once + the live requests' cache) over its time, against 8 TB/s; ``points`` = decode at batch 1 and
64.  The reference publishes no number for this configuration, so ``vs_baseline`` is null.
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

QWEN3_8B = dict(architectures=["Qwen3ForCausalLM"], hidden_size=4096, num_hidden_layers=36,
                num_attention_heads=32, num_key_value_heads=8, head_dim=128, intermediate_size=12288,
                vocab_size=151936, rope_theta=1000000.0, rms_norm_eps=1e-6, max_position_embeddings=40960,
                tie_word_embeddings=False, attention_bias=False, use_sliding_window=False,
                initializer_range=0.02, torch_dtype="bfloat16")

# the reference's own benchmark (bench.py:10-45, README.md:129-147): Qwen3-0.6B, 256 requests, prompt and
# generation lengths uniform in 100..1024, temperature 0.6, no end-of-sequence; 9032.37 tokens/s on an A100 40GB
QWEN3_0P6B = dict(architectures=["Qwen3ForCausalLM"], hidden_size=1024, num_hidden_layers=28,
                  num_attention_heads=16, num_key_value_heads=8, head_dim=128, intermediate_size=3072,
                  vocab_size=151936, rope_theta=1000000.0, rms_norm_eps=1e-6, max_position_embeddings=40960,
                  tie_word_embeddings=True, attention_bias=False, use_sliding_window=False,
                  initializer_range=0.02, torch_dtype="bfloat16")
REFERENCE_MIXED_TOK_S = 9032.37
QWEN3_14B = dict(QWEN3_8B, hidden_size=5120, num_hidden_layers=40, num_attention_heads=40, intermediate_size=17408)
QWEN3_32B = dict(QWEN3_8B, hidden_size=5120, num_hidden_layers=64, num_attention_heads=64, intermediate_size=25600)
SIZES = {"0.6b": QWEN3_0P6B, "8b": QWEN3_8B, "14b": QWEN3_14B, "32b": QWEN3_32B}


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
    ap.add_argument("--no-points", action="store_true", help="skip the batch 1 / 64 points and the prefill")
    ap.add_argument("--eager", action="store_true", help="no HIP graphs")
    ap.add_argument("--size", choices=sorted(SIZES), default=None,
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


def run_mixed(dtype, eager, size="0.6b"):
    """Output tokens per second over 256 requests arriving at once, continuous batching; returns
    (tokens/s, output tokens, seconds, engine steps)."""
    import random
    import torch
    from ullm_amd import EngineConfig, SamplingParams
    from ullm_amd.engine.engine import Engine
    from ullm_amd.engine.loading import make_env
    from ullm_amd.models import build_model
    from ullm_amd.weights.random_init import bind_random_weights

    cfg, model = build_model(dict(SIZES[size]))
    env = make_env(dtype, "cuda:0", 4096)
    bind_random_weights(model, env, seed=0)
    rng = random.Random(0)
    n = 256
    prompts = [[rng.randint(0, 10000) for _ in range(rng.randint(100, 1024))] for _ in range(n)]
    new_tokens = [rng.randint(100, 1024) for _ in range(n)]
    ec = EngineConfig(model="(random)", dtype=dtype, max_bs=256, context_len=4096, page_size=16,
                      num_pages=n * 130, max_num_batched_tokens=8192, max_prefill_chunk=2048, enforce_eager=eager)
    eng = Engine(ec, model=model, env=env, model_config=cfg)
    eng.add_request("warm", prompts[0][:64], SamplingParams(temperature=0.6, ignore_eos=True, max_new_tokens=10))
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


def main():
    args = parse_args()
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported")
        return 2
    import torch
    from ullm_amd import EngineConfig, SamplingParams
    from ullm_amd.engine.engine import Engine
    from ullm_amd.engine.loading import make_env
    from ullm_amd.models import build_model
    from ullm_amd.weights.random_init import bind_random_weights

    if args.mixed_only:
        size = args.size or "0.6b"
        tok_s, n_out, secs, steps = run_mixed(args.dtype, args.eager, size)
        print(json.dumps({"metric": f"output tok/s, 256 requests, lengths 100..1024 in and out, Qwen3-{size} sizes",
                          "value": round(tok_s, 1), "unit": "tokens/s", "output_tokens": n_out,
                          "seconds": round(secs, 3), "engine_steps": steps,
                          "vs_baseline": round(tok_s / REFERENCE_MIXED_TOK_S, 3) if size == "0.6b" else None,
                          "baseline": "9032.37 tokens/s, the reference with Qwen3-0.6B on an A100 40GB"}))
        return 0
    args.size = args.size or "8b"
    config = dict(SIZES[args.size])
    full_layers = config["num_hidden_layers"]
    if args.layers is not None:
        config["num_hidden_layers"] = args.layers
    cfg, model = build_model(config)
    env = make_env(args.dtype, "cuda:0", args.context_len)
    bind_random_weights(model, env, seed=0)
    itemsize = 2 if args.dtype == "bfloat16" else 4
    wbytes = weight_bytes(model, itemsize)
    kv_per_token = sum(g.bytes_per_token(itemsize) for g in model.cache_layout()[0])
    gen = torch.Generator().manual_seed(0)

    def run_decode(batch, steps, warmup, top_k=-1, top_p=1.0):
        """tokens/s, ms per step, bytes read per step (mean over the timed steps)."""
        budget = max(8192, batch)
        # requests that finish their prompt early decode while the others are still in theirs
        new_tokens = warmup + steps + 4 + -(-batch * args.prompt_len // budget)
        ec = EngineConfig(model="(random)", dtype=args.dtype, max_bs=batch, context_len=args.context_len,
                          page_size=16, num_pages=batch * (-(-(args.prompt_len + new_tokens + 16) // 16)),
                          max_num_batched_tokens=budget, max_prefill_chunk=2048, enforce_eager=args.eager)
        eng = Engine(ec, model=model, env=env, model_config=cfg)
        for i in range(batch):
            prompt = torch.randint(0, cfg.vocab_size, (args.prompt_len,), generator=gen).tolist()
            eng.add_request(f"r{i}", prompt, SamplingParams(temperature=0.6, top_k=top_k, top_p=top_p, ignore_eos=True,
                                                            seed=i, max_new_tokens=new_tokens))
        while any(r.num_computed < args.prompt_len for r in eng.scheduler.requests.values()) or eng.scheduler.waiting:
            eng.step()                                   # prefill (untimed)
        for _ in range(warmup):
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
        return batch * steps / dt, dt / steps * 1e3, wbytes + kv_per_token * mean_ctx

    def run_prefill(n_tokens):
        ec = EngineConfig(model="(random)", dtype=args.dtype, max_bs=1, context_len=args.context_len, page_size=16,
                          num_pages=-(-(n_tokens + 16) // 16), max_num_batched_tokens=n_tokens,
                          max_prefill_chunk=n_tokens, enforce_eager=True)
        eng = Engine(ec, model=model, env=env, model_config=cfg)
        best = None
        for rep in range(4):
            prompt = torch.randint(0, cfg.vocab_size, (n_tokens,), generator=gen).tolist()
            eng.add_request(f"p{rep}", prompt, SamplingParams(temperature=0.0, max_new_tokens=1, ignore_eos=True))
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
        flops = step_flops(cfg, n_tokens, n_tokens * (n_tokens + 1) // 2, 1)
        return n_tokens / best, best * 1e3, flops / best / PEAK_FLOPS[args.dtype]

    if args.prefill_only:
        p_tok_s, p_ms, p_frac = run_prefill(args.prefill_only)
        print(json.dumps({"prefill": {"value": round(p_tok_s, 1), "tokens": args.prefill_only, "ms": round(p_ms, 3),
                                      "frac": round(p_frac, 4)}}))
        return 0
    tok_s, ms, bytes_step = run_decode(args.batch, args.steps, args.warmup, args.top_k, args.top_p)
    achieved = bytes_step / (ms * 1e-3) / 1e9
    line = {
        "metric": f"decode tok/s at bs {args.batch} (also bs 1/64, prefill tok/s at 2048; % of roofline), Qwen3-{args.size}",
        "value": round(tok_s, 2), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32", "data": "synthetic",
        "config": {"model": f"Qwen3-{args.size} sizes, random weights", "layers": config["num_hidden_layers"],
                   "layers_of_config": full_layers, "hidden_size": cfg.hidden_size,
                   "num_attention_heads": cfg.num_attention_heads, "num_key_value_heads": cfg.num_key_value_heads,
                   "head_dim": cfg.head_dim, "intermediate_size": cfg.intermediate_size, "vocab_size": cfg.vocab_size,
                   "global_batch": args.batch, "prompt_len": args.prompt_len, "seq_len": args.context_len,
                   "page_size": 16, "sampling": "temperature 0.6, seeded" + (f", top-k {args.top_k}" if args.top_k > 0 else "") + (f", top-p {args.top_p}" if args.top_p < 1 else ""), "parallelism": "single GPU",
                   "hip_graphs": not args.eager},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4)},
    }
    if not args.no_points:
        p_tok_s, p_ms, p_frac = run_prefill(2048)
        line["prefill"] = {"value": round(p_tok_s, 1), "tokens": 2048, "ms": round(p_ms, 3), "frac": round(p_frac, 4)}
        b1, _, _ = run_decode(1, min(args.steps, 32), min(args.warmup, 4))
        b64, _, _ = run_decode(64, min(args.steps, 32), min(args.warmup, 4))
        # the same batch with the sampling of Qwen3's generation_config.json (top-k 20, top-p 0.95)
        b8f, _, _ = run_decode(args.batch, args.steps, args.warmup, top_k=20, top_p=0.95)
        line["points"] = {"decode_b1": round(b1, 2), "decode_b64": round(b64, 2),
                          f"decode_b{args.batch}_top_k20_top_p95": round(b8f, 2)}
        del model
        torch.cuda.empty_cache()
        m_tok_s, m_out, m_secs, _ = run_mixed(args.dtype, args.eager)
        # the reference's own benchmark (Qwen3-0.6B, 256 requests); its 9032.37 tokens/s are from an A100 40GB
        line["mixed_qwen3_0p6b"] = {"value": round(m_tok_s, 1), "unit": "output tokens/s", "output_tokens": m_out,
                                    "seconds": round(m_secs, 3),
                                    "vs_reference_a100": round(m_tok_s / REFERENCE_MIXED_TOK_S, 3)}
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
