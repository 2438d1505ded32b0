"""y = x W^T (+ b) with W stored [out, in] as the reference's linears are
(ullm/layers/linear.py:165,268).  The float32 mode always takes the hand-written 32-bit kernel
(fixed K order, no matrix-core input rounding); bfloat16 takes the skinny weight-streaming kernel
for few rows and the library product for many, as the reference uses a library product throughout.
"""
from __future__ import annotations

from typing import Optional

import torch

from ..kernels import ops


def linear(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None,
           out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    out_dtype = out_dtype or x.dtype
    if x.dtype == torch.float32 or weight.dtype == torch.float32:
        return ops.gemm_simple(x, weight, bias, out_dtype=out_dtype)
    return ops.gemm_bf16(x, weight, bias, out_dtype=out_dtype)
