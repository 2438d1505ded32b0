"""Plain, slow implementation of the Qwen3 dense decoder and of the sampler, written from the
reference's formulas: whole sequences, no cache, no batching, one function per part, float32
torch on the CPU.  It shares no code with ``ullm_amd``: it reads config.json as a dict and the
safetensors file with the safetensors library directly.

Citations are file:line in the reference tree (ullm/...).
"""
from __future__ import annotations

import json
import math
import os
from typing import Dict, List, Optional

import torch


# ---------------------------------------------------------------------------- parts

def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """ullm/layers/layernorm.py:23,28-30: x32 * rsqrt(mean(x32^2, -1) + eps) * weight."""
    x = x.to(torch.float32)
    variance = x.pow(2).mean(dim=-1, keepdim=True)
    return x * torch.rsqrt(variance + eps) * weight.to(torch.float32)


def rope_cos_sin(positions: torch.Tensor, rotary_dim: int, base: float):
    """ullm/layers/rotary_embedding.py:52-75: inv_freq_i = 1 / base^(2i/d), angle = p * inv_freq,
    in float32; returns cos, sin of shape [T, d/2]."""
    inv_freq = 1.0 / (base ** (torch.arange(0, rotary_dim, 2, dtype=torch.float) / rotary_dim))
    t = positions.to(torch.float)
    freqs = torch.einsum("i,j -> ij", t, inv_freq)
    return freqs.cos(), freqs.sin()


def apply_rope_reference_layout(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """ullm/layers/rotary_embedding.py:5-24 exactly: halves x1 = x[..., :d/2], x2 = x[..., d/2:];
    o1 = x1 cos - x2 sin, o2 = x2 cos + x1 sin; output = stack((o1, o2), -1).flatten(-2), which puts
    o1[i] at 2i and o2[i] at 2i+1.  x: [T, heads, d]; cos, sin: [T, d/2]."""
    cos = cos.unsqueeze(-2)
    sin = sin.unsqueeze(-2)
    x1, x2 = torch.chunk(x, 2, dim=-1)
    o1 = x1 * cos - x2 * sin
    o2 = x2 * cos + x1 * sin
    return torch.stack((o1, o2), dim=-1).flatten(-2)


def apply_rope_concat_layout(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """The same rotation with o1 and o2 concatenated instead of interleaved.  Query and key get the
    same fixed permutation of the head dimension either way, so every q.k is unchanged."""
    cos = cos.unsqueeze(-2)
    sin = sin.unsqueeze(-2)
    x1, x2 = torch.chunk(x, 2, dim=-1)
    return torch.cat((x1 * cos - x2 * sin, x2 * cos + x1 * sin), dim=-1)


def causal_gqa_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float,
                         window: int = 0) -> torch.Tensor:
    """Attention of one whole sequence.  q: [T, nq, d]; k, v: [T, nkv, d].
    scale = head_dim^-0.5 (ullm/models/qwen3.py:81, passed as sm_scale ullm/layers/attention.py:305);
    causal=True (attention.py:88); query head h reads kv head h // (nq // nkv) (attention.py:271,
    contiguous groups as the q/kv sharding of ullm/layers/linear.py:394-399 implies).
    ``window`` > 0 keeps only keys j with i - window < j <= i (the reference never windows; 0 = its
    behaviour)."""
    T, nq, d = q.shape
    nkv = k.shape[1]
    group = nq // nkv
    out = torch.empty_like(q)
    i = torch.arange(T).unsqueeze(1)
    j = torch.arange(T).unsqueeze(0)
    allowed = j <= i
    if window > 0:
        allowed = allowed & (j > i - window)
    for h in range(nq):
        kh = h // group
        s = (q[:, h, :] @ k[:, kh, :].T) * scale
        s = s.masked_fill(~allowed, float("-inf"))
        p = torch.softmax(s, dim=-1)
        out[:, h, :] = p @ v[:, kh, :]
    return out


def silu_and_mul(x: torch.Tensor) -> torch.Tensor:
    """ullm/layers/activation.py:16-18: silu(x[..., :d]) * x[..., d:]."""
    d = x.shape[-1] // 2
    return torch.nn.functional.silu(x[..., :d]) * x[..., d:]


def linear(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """ullm/layers/linear.py:165,268: F.linear(x, W[out, in], bias)."""
    y = x @ weight.to(torch.float32).T
    if bias is not None:
        y = y + bias.to(torch.float32)
    return y


# ---------------------------------------------------------------------------- layers

def qwen3_attention(x, positions, w: Dict[str, torch.Tensor], prefix: str, cfg: dict, window: int):
    """ullm/models/qwen3.py:113-130: qkv projection, split, per-head q/k RMS norm with one gain of
    size head_dim shared by all heads (qwen3.py:110-111,121-126), rotation (qwen3.py:127), attention,
    output projection without bias (qwen3.py:91-95,129)."""
    nq, nkv = cfg["num_attention_heads"], cfg["num_key_value_heads"]
    d = cfg.get("head_dim") or cfg["hidden_size"] // nq
    eps = cfg["rms_norm_eps"]
    T = x.shape[0]
    bias = (lambda n: w.get(f"{prefix}.{n}.bias")) if cfg.get("attention_bias", False) else (lambda n: None)
    q = linear(x, w[f"{prefix}.q_proj.weight"], bias("q_proj")).view(T, nq, d)
    k = linear(x, w[f"{prefix}.k_proj.weight"], bias("k_proj")).view(T, nkv, d)
    v = linear(x, w[f"{prefix}.v_proj.weight"], bias("v_proj")).view(T, nkv, d)
    q = rms_norm(q, w[f"{prefix}.q_norm.weight"], eps)
    k = rms_norm(k, w[f"{prefix}.k_norm.weight"], eps)
    cos, sin = rope_cos_sin(positions, d, float(cfg.get("rope_theta", 1000000)))
    q = apply_rope_reference_layout(q, cos, sin)
    k = apply_rope_reference_layout(k, cos, sin)
    o = causal_gqa_attention(q, k, v, d ** -0.5, window)
    return linear(o.reshape(T, nq * d), w[f"{prefix}.o_proj.weight"])


def qwen3_mlp(x, w: Dict[str, torch.Tensor], prefix: str):
    """ullm/models/qwen3.py:42-46 with gate_up rows = gate then up (qwen3.py:307-308)."""
    gate_up = torch.cat((linear(x, w[f"{prefix}.gate_proj.weight"]),
                         linear(x, w[f"{prefix}.up_proj.weight"])), dim=-1)
    return linear(silu_and_mul(gate_up), w[f"{prefix}.down_proj.weight"])


def window_of_layer(cfg: dict, layer: int) -> int:
    """The reference reads none of the sliding-window keys (0 everywhere).  When a config switches
    ``use_sliding_window`` on, layers from ``max_window_layers`` on look back ``sliding_window``
    keys, the current one included; a list ``layer_types`` names the layers that do instead."""
    if not cfg.get("use_sliding_window", False):
        return 0
    if cfg.get("layer_types"):
        return int(cfg["sliding_window"]) if cfg["layer_types"][layer] == "sliding_attention" else 0
    return int(cfg["sliding_window"]) if layer >= cfg.get("max_window_layers", cfg["num_hidden_layers"]) else 0


def qwen3_forward(w: Dict[str, torch.Tensor], cfg: dict, token_ids: List[int]) -> torch.Tensor:
    """Logits [T, vocab] of one whole sequence.

    ullm/models/qwen3.py:228-255 and :159-178: h = embed(ids); per layer the residual is carried
    beside the branch output: (x, res) = norm_in(h, res) means res <- h + res and x = norm(res);
    after attention (x, res) = norm_post(attn, res); the layer returns (mlp(x), res); after the last
    layer x = norm_final(mlp_out, res).  That is h <- h + attn(norm(h)); h <- h + mlp(norm(h));
    out = norm(h).  Logits = out @ lm_head^T (ullm/layers/vocab_parallel_embedding.py:158-162),
    lm_head being the embedding when the checkpoint ties them.
    """
    w = {k: v.to(torch.float32) for k, v in w.items()}
    ids = torch.tensor(token_ids, dtype=torch.long)
    positions = torch.arange(len(token_ids))
    eps = cfg["rms_norm_eps"]
    h = w["model.embed_tokens.weight"][ids]
    for layer in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{layer}"
        x = rms_norm(h, w[f"{p}.input_layernorm.weight"], eps)
        h = h + qwen3_attention(x, positions, w, f"{p}.self_attn", cfg, window_of_layer(cfg, layer))
        x = rms_norm(h, w[f"{p}.post_attention_layernorm.weight"], eps)
        h = h + qwen3_mlp(x, w, f"{p}.mlp")
    x = rms_norm(h, w["model.norm.weight"], eps)
    head = w.get("lm_head.weight")
    if head is None:
        if not cfg.get("tie_word_embeddings", False):
            raise KeyError("lm_head.weight is absent and tie_word_embeddings is false")
        head = w["model.embed_tokens.weight"]
    return linear(x, head)


def load_model_folder(model_dir: str):
    from safetensors.torch import load_file
    with open(os.path.join(model_dir, "config.json")) as f:
        cfg = json.load(f)
    w = {}
    for name in sorted(os.listdir(model_dir)):
        if name.endswith(".safetensors"):
            w.update(load_file(os.path.join(model_dir, name)))
    return cfg, w


# ---------------------------------------------------------------------------- sampling

def uniform_from_seed(seed: int, position: int) -> float:
    """The engine's counter-based uniform in [0, 1): splitmix64 of (seed, position), top 24 bits."""
    mask = (1 << 64) - 1
    z = (seed * 0x9E3779B97F4A7C15 + (position + 1) * 0xD1B54A32D192ED03) & mask
    z = (z + 0x9E3779B97F4A7C15) & mask
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & mask
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & mask
    z = z ^ (z >> 31)
    return (z >> 40) / float(1 << 24)


def filter_logits(logits: torch.Tensor, temperature: float, top_k: int, top_p: float, min_p: float):
    """ullm/layers/sampler.py:39-47 on one row: divide by the temperature (<= 0 -> 1.0, :40-42),
    top-k on the ascending sort (k <= 0 -> all; entries below the k-th largest value -> -inf, :67-76),
    top-p (p <= 0 -> 1; mask where the ascending cumulative probability <= 1 - p, last never, :78-92),
    min-p (probabilities below min_p * max -> -inf, :95-107)."""
    x = logits.to(torch.float32).clone()
    t = 1.0 if temperature <= 0 else temperature
    x = x / t
    V = x.numel()
    xs, idx = x.sort(descending=False)
    k = V if top_k <= 0 else min(top_k, V)
    thresh = xs[V - k]
    xs = xs.masked_fill(xs < thresh, float("-inf"))
    p = 1.0 if top_p <= 0 else top_p
    probs = xs.softmax(dim=-1)
    cum = probs.cumsum(dim=-1)
    mask = cum <= 1 - p
    mask[-1] = False
    xs = xs.masked_fill(mask, float("-inf"))
    x = torch.empty_like(xs).scatter_(0, idx, xs)
    probs = torch.softmax(x, dim=-1)
    x = x.masked_fill(probs < min_p * probs.max(), float("-inf"))
    return x


def sample_token(logits: torch.Tensor, temperature: float, top_k: int, top_p: float, min_p: float,
                 seed: int, position: int) -> int:
    """Greedy when temperature == 0 (first index of the maximum); else the filtered distribution
    (softmax, ullm/layers/sampler.py:49) drawn by inverse CDF in index order with the seeded uniform
    instead of the reference's unseeded torch.multinomial (sampler.py:56)."""
    if temperature == 0:
        return int(torch.argmax(logits.to(torch.float32)).item())
    x = filter_logits(logits, temperature, top_k, top_p, min_p)
    probs = torch.softmax(x.double(), dim=-1)
    cdf = probs.cumsum(dim=-1)
    u = uniform_from_seed(seed, position) * float(cdf[-1])
    tok = int(torch.searchsorted(cdf, torch.tensor(u, dtype=cdf.dtype), right=True).item())
    keep = torch.nonzero(probs > 0).flatten()
    tok = min(tok, int(keep[-1]))
    while probs[tok] == 0:
        tok += 1
    return tok


def sample_token_set(logits: torch.Tensor, temperature: float, top_k: int, top_p: float, min_p: float,
                     seed: int, position: int, slack: float = 2e-5) -> set:
    """The tokens an inverse-CDF draw may give when the sums are taken in 32-bit in another order:
    every kept token whose CDF interval comes within ``slack`` of the seeded uniform.  Almost always
    one token (the one :func:`sample_token` returns); two when the draw falls on a boundary."""
    if temperature == 0:
        return {sample_token(logits, temperature, top_k, top_p, min_p, seed, position)}
    probs = torch.softmax(filter_logits(logits, temperature, top_k, top_p, min_p).double(), dim=-1)
    cdf = probs.cumsum(dim=-1)
    u = uniform_from_seed(seed, position) * float(cdf[-1])
    lower = cdf - probs
    near = (probs > 0) & (lower - slack <= u) & (u < cdf + slack)
    return set(torch.nonzero(near).flatten().tolist()) | {sample_token(logits, temperature, top_k, top_p, min_p,
                                                                        seed, position)}


def greedy_generate(w, cfg, prompt: List[int], n_new: int) -> List[int]:
    ids = list(prompt)
    for _ in range(n_new):
        ids.append(int(torch.argmax(qwen3_forward(w, cfg, ids)[-1]).item()))
    return ids[len(prompt):]
