"""Grouped-query attention over the paged cache, as a mixer.

Reference: ullm/models/qwen3.py:49-130 (projection, per-head q/k norm, rotation, attention, output
projection) and ullm/layers/attention.py:279-313 (write k, v to the cache, then attend over it).
Head size is a parameter of its own (qwen3.py:78: not hidden/heads), the q/k norms and the position
encoding are optional parts, and a window bounds how far back a query looks (0 = everything; the
reference never windows).
"""
from __future__ import annotations

from typing import Dict, List, Optional

import numpy as np
import torch

from ..kernels import ops
from .base import (KVNeed, LayerCache, Mixer, PartEnv, PositionEncoding, StepContext, StepPlan, StepShape, WeightDecl,
                   register_part)
from .linear import add_into_stream, can_fuse, linear, linear_into_stream, linear_of_norm


# Up to this many single new tokens a step, the attention kernel norms, rotates and writes the new keys itself.
# With more, its waves fill the chip and the extra work at each wave's start is no longer hidden behind the
# others' loads: the kernel of its own, which does it for all tokens at once, is then the faster way.
FUSED_DECODE_MAX_TOKENS = 64


def plan_attention_step(shape: StepShape) -> StepPlan:
    """How the attention kernels split a batch: the tokens of one-token entries (``decode_tokens``, longest
    context first: the short ones fill the tail of the launch), and tiles of up to ``ops.PREFILL_TILE``
    consecutive tokens (first token, count) of the longer entries by rising number of keys (``tiles``), with
    the numbers the launches are shaped by.  Padding entries of a captured batch are one-token entries."""
    dec, tiles, max_decode_kv, t0 = [], [], 0, 0
    for n, start in zip(shape.lens, shape.starts):
        if n == 1:
            dec.append((-start, t0))
            max_decode_kv = max(max_decode_kv, start + 1)
        else:
            for first in range(0, n, ops.PREFILL_TILE):
                count = min(ops.PREFILL_TILE, n - first)
                tiles.append((start + first + count, t0 + first, count))
        t0 += n
    tiles.sort()
    dec.sort()
    decode_tokens = [t for _, t in dec] + list(range(t0, t0 + shape.pad_entries))
    if shape.kv_bucket is not None:
        max_decode_kv = shape.kv_bucket                   # a captured launch: the split of the keys is fixed
    return StepPlan(
        arrays={"decode_tokens": np.asarray(decode_tokens, dtype=np.int32),
                "tiles": np.asarray([x for _, first, count in tiles for x in (first, count)], dtype=np.int32)},
        facts={"num_decode": len(decode_tokens), "max_decode_kv": max_decode_kv, "num_tiles": len(tiles),
               "tile_keys_total": sum(k for k, _, _ in tiles), "tile_keys_max": tiles[-1][0] if tiles else 0})


@register_part("mixer", "gqa_attention")
class GQAttention(Mixer):
    folds_norm = True
    hands_norm_ahead = True
    step_planners = {"attention": plan_attention_step}

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int, prefix: str,
                 position: Optional[PositionEncoding] = None, qk_norm_eps: Optional[float] = None,
                 bias: bool = False, window: int = 0, scale: Optional[float] = None):
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} query heads are not a multiple of {num_kv_heads} kv heads")
        if head_dim % 2 or head_dim > 512:
            raise ValueError(f"head_dim={head_dim} must be even and at most 512")
        self.hidden_size, self.nq, self.nkv, self.hd = hidden_size, num_heads, num_kv_heads, head_dim
        self.prefix = prefix
        self.position = position
        self.qk_norm_eps = qk_norm_eps          # None: no per-head norm
        self.bias = bias
        self.window = int(window)
        self.scale = float(scale) if scale is not None else head_dim ** -0.5   # qwen3.py:81
        self.w_qkv = self.b_qkv = self.w_o = self.q_gain = self.k_gain = None

    def children(self):
        return [self.position] if self.position is not None else []

    def cache_need(self):
        return KVNeed(self.nkv, self.hd, self.window)

    def weights(self) -> List[WeightDecl]:
        p, H, hd = self.prefix, self.hidden_size, self.hd
        # q, k and v are used as one matrix with rows q | k | v, as the reference merges them
        # (ullm/layers/linear.py:381-389); the loader puts the three tensors into its rows
        rows = (("q", self.nq * hd, 0), ("k", self.nkv * hd, self.nq * hd), ("v", self.nkv * hd, (self.nq + self.nkv) * hd))
        out = [WeightDecl(f"{p}.{n}_proj.weight", (r, H), merged_into=f"{p}.qkv_proj.weight", row_offset=off)
               for n, r, off in rows]
        out.append(WeightDecl(f"{p}.o_proj.weight", (H, self.nq * hd)))
        if self.bias:   # qwen3.py:146 (attention_bias): on q, k, v only; o_proj never has one (qwen3.py:94)
            out += [WeightDecl(f"{p}.{n}_proj.bias", (r,), keep_fp32=True, merged_into=f"{p}.qkv_proj.bias", row_offset=off)
                    for n, r, off in rows]
        if self.qk_norm_eps is not None:
            out += [WeightDecl(f"{p}.q_norm.weight", (hd,), init="gain", keep_fp32=True),
                    WeightDecl(f"{p}.k_norm.weight", (hd,), init="gain", keep_fp32=True)]
        return out

    def bind(self, tensors: Dict[str, torch.Tensor], env: PartEnv) -> None:
        p = self.prefix
        self.w_qkv = tensors[f"{p}.qkv_proj.weight"].contiguous()
        self.w_o = tensors[f"{p}.o_proj.weight"].contiguous()
        if self.bias:
            self.b_qkv = tensors[f"{p}.qkv_proj.bias"].contiguous()
        if self.qk_norm_eps is not None:
            self.q_gain = tensors[f"{p}.q_norm.weight"].contiguous()
            self.k_gain = tensors[f"{p}.k_norm.weight"].contiguous()

    def forward(self, x: torch.Tensor, ctx: StepContext, cache: LayerCache) -> torch.Tensor:
        return linear_into_stream(self._attend(linear(x, self.w_qkv, self.b_qkv), ctx, cache), self.w_o, ctx)

    def fusable(self, residual, ctx: StepContext) -> bool:
        return can_fuse(residual, ctx.dtype, self.w_qkv, self.w_o)

    def forward_fused(self, x, residual, ctx: StepContext, cache: LayerCache, then=None):
        qkv = linear_of_norm(x, self.w_qkv, self.b_qkv)                               # the norm before folded in
        # the residual add, and the next norm's share of the work, folded behind
        return add_into_stream(self._attend(qkv, ctx, cache), self.w_o, residual, then, ctx.dtype)

    def _attend(self, qkv: torch.Tensor, ctx: StepContext, cache: LayerCache) -> torch.Tensor:
        """Per-head norm, rotation, cache write and attention for a fused projection [T, (nq+2nkv)*hd];
        returns the heads' outputs [T, nq*hd]."""
        T = qkv.shape[0]
        x = qkv
        group = ctx.groups[cache.group]
        table, rot, style = self.position.kernel_args() if self.position is not None else (None, 0, 0)
        eps = self.qk_norm_eps if self.qk_norm_eps is not None else 0.0
        plan = ctx.plans["attention"]
        work = plan.facts
        if (work["num_decode"] == T and not work["num_tiles"] and T <= FUSED_DECODE_MAX_TOKENS
                and ops.attention_decode_fused_supports(x.dtype, self.hd, group.page_size, self.nq, self.nkv, rot, style)):
            # a step of single new tokens: norm, rotation and cache write happen inside the attention kernel
            out = torch.empty((T, self.nq * self.hd), dtype=x.dtype, device=x.device)
            ops.attention_decode_fused(
                qkv, out, self.q_gain, self.k_gain, eps, table, rot, style, cache.k_pool, cache.v_pool,
                plan.arrays["decode_tokens"], work["num_decode"], ctx.positions, ctx.token_entry, group.block_table,
                group.page_size, self.nq, self.nkv, self.hd, self.scale, self.window, work["max_decode_kv"],
                write_kv=cache.owner)
            return out
        q = torch.empty((T, self.nq * self.hd), dtype=x.dtype, device=x.device)
        ops.qk_norm_rope_write(
            qkv, q, self.q_gain, self.k_gain, eps,
            table, rot, style, ctx.positions, ctx.token_entry, group.block_table,
            cache.k_pool, cache.v_pool, group.page_size, self.nq, self.nkv, self.hd, write_kv=cache.owner)
        return ops.paged_attention(q, cache.k_pool, cache.v_pool, ctx, group, self.nq, self.nkv, self.hd,
                                   self.scale, self.window, plan)
