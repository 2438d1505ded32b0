"""RMS norm fused with the residual add (reference: ullm/layers/layernorm.py:15-34).

The reference carries the residual in the model dtype and rounds the 32-bit sum once per add
(layernorm.py:25-26); here the residual stream itself stays 32-bit, so the sum is never rounded.
The gain is held in 32-bit (the reference promotes it for the multiply, layernorm.py:30).
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..kernels import ops
from .base import Norm, PartEnv, PendingNorm, WeightDecl, register_part


@register_part("norm", "rmsnorm")
class RMSNorm(Norm):
    adds_stacks = True

    def __init__(self, size: int, eps: float, weight_name: str):
        self.size = size
        self.eps = float(eps)
        self.weight_name = weight_name
        self.gain: Optional[torch.Tensor] = None

    def weights(self) -> List[WeightDecl]:
        return [WeightDecl(self.weight_name, (self.size,), init="gain", keep_fp32=True)]

    def bind(self, tensors: Dict[str, torch.Tensor], env: PartEnv) -> None:
        self.gain = tensors[self.weight_name].contiguous()

    def add_norm(self, branch, residual, rows=None, out_dtype=None):
        if out_dtype is None:
            out_dtype = branch.dtype if branch is not None and branch.dim() == 2 else torch.float32
        return ops.add_rmsnorm(branch, residual, self.gain, self.eps, out_dtype, rows=rows)

    def pending(self, residual, out_dtype, scaled=None, squares=None):
        return PendingNorm(self, residual, self.gain, self.eps, out_dtype, scaled, squares)

    def ahead_gain(self):
        return self.gain
