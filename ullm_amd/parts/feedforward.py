"""Dense gated feed-forward: down(silu(gate(x)) * up(x)), no biases
(ullm/models/qwen3.py:23-46, ullm/layers/activation.py:16-18).  gate and up are one fused
projection with rows gate | up (qwen3.py:307-308).
"""
from __future__ import annotations

from typing import Dict, List

import torch

from ..kernels import ops
from .base import FeedForward, PartEnv, StepContext, WeightDecl, register_part
from .linear import add_into_stream, can_fuse, gate_up, linear_into_stream, linear_of_norm


@register_part("ffn", "swiglu")
class SwiGLU(FeedForward):
    folds_norm = True
    hands_norm_ahead = True

    def __init__(self, hidden_size: int, intermediate_size: int, prefix: str):
        self.hidden_size, self.intermediate_size, self.prefix = hidden_size, intermediate_size, prefix
        self.w_gate_up = self.w_down = None

    def weights(self) -> List[WeightDecl]:
        p, H, I = self.prefix, self.hidden_size, self.intermediate_size
        merged = f"{p}.gate_up_proj.weight"          # rows gate | up, put together by the loader
        return [WeightDecl(f"{p}.gate_proj.weight", (I, H), merged_into=merged, row_offset=0),
                WeightDecl(f"{p}.up_proj.weight", (I, H), merged_into=merged, row_offset=I),
                WeightDecl(f"{p}.down_proj.weight", (H, I))]

    def bind(self, tensors: Dict[str, torch.Tensor], env: PartEnv) -> None:
        p = self.prefix
        self.w_gate_up = tensors[f"{p}.gate_up_proj.weight"].contiguous()
        self.w_down = tensors[f"{p}.down_proj.weight"].contiguous()

    def forward(self, x: torch.Tensor, ctx: StepContext) -> torch.Tensor:
        act = gate_up(x, self.w_gate_up)
        return linear_into_stream(act, self.w_down, ctx)

    def fusable(self, residual, ctx: StepContext) -> bool:
        return can_fuse(residual, ctx.dtype, self.w_gate_up, self.w_down)

    def forward_fused(self, x, residual, ctx: StepContext, then=None):
        act = linear_of_norm(x, self.w_gate_up, silu=True)     # the norm before, silu(gate) * up behind the first product
        return add_into_stream(act, self.w_down, residual, then, ctx.dtype)   # residual add (and the next norm's part) behind the second
