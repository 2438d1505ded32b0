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


# Rows up to which folding the norm into the product pays: beyond, the float32 rows of X cost every block more
# registers and loads than the saved launch is worth.  A small matrix (q|k|v of the 8B and 14B sizes) has few
# blocks to pay that price, and the launch of the norm's own kernel weighs more beside its short product: there
# the norm is folded in for every row count the kernel takes.
NORM_FOLDED_MAX_ROWS = 8
NORM_FOLDED_SMALL_WEIGHT = 40 << 20     # elements


def linear_of_norm(x, weight: torch.Tensor, bias: Optional[torch.Tensor] = None, silu: bool = False) -> torch.Tensor:
    """The first projection of a part whose input may be a norm not yet computed
    (:class:`~ullm_amd.parts.base.PendingNorm`): then the norm is folded into the product where the
    kernel takes the shapes, and computed first where not.  With ``silu`` the weights are gate | up
    and the result silu(gate) * up."""
    from .base import PendingNorm
    if isinstance(x, PendingNorm):
        if (x.out_dtype == torch.bfloat16
                and (x.stream.shape[0] <= NORM_FOLDED_MAX_ROWS or weight.numel() <= NORM_FOLDED_SMALL_WEIGHT)
                and ops.gemm_skinny_normed_supports(x.stream, x.gain, weight)):
            return ops.gemm_skinny_normed(x.stream, x.gain, x.eps, weight, bias, silu=silu)
        x = x.apply()
    if silu:
        return ops.gemm_skinny_silu(x, weight)
    return linear(x, weight, bias)


FUSED_MAX_ROWS = 16      # batches up to this many tokens take the projections with the folded add / activation


def can_fuse(residual: torch.Tensor, dtype: torch.dtype, *weights: torch.Tensor) -> bool:
    """True if the folded projection kernels take this batch: bfloat16 compute, few rows, row lengths
    that keep 16-byte alignment."""
    T, H = residual.shape
    if dtype != torch.bfloat16 or T > FUSED_MAX_ROWS or H % 8:
        return False
    return all(w.dtype == torch.bfloat16 and w.shape[1] % 8 == 0 and w.shape[0] % 4 == 0 and w.data_ptr() % 16 == 0
               for w in weights)


STACKED_MIN_ROWS, STACKED_MAX_ROWS = 17, 256
# smallest matrix (elements) that goes this way: below (Qwen3-0.6B's projections, 2-3 M elements), the stack the
# norm has to read outweighs the matrix
STACKED_MIN_WEIGHT = 8 << 20


def linear_into_stream(x: torch.Tensor, weight: torch.Tensor, ctx) -> torch.Tensor:
    """The last projection of a mixer or feed-forward, whose result the next norm adds to the residual
    stream.  For 17 to 256 rows in bfloat16, where the model's norms add stacks, it is a stack of
    float32 partial sums over slices of the inner dimension (the slices fill the chip, the norm adds
    them in order); otherwise the plain product.  For few long rows the library's choice of kernel
    is two to five times off the memory roofline at these row counts."""
    if (ctx.stacked_branches and x.dtype == torch.bfloat16 and STACKED_MIN_ROWS <= x.shape[0] <= STACKED_MAX_ROWS
            and weight.numel() >= STACKED_MIN_WEIGHT and ops.gemm_partial_sums_supports(x, weight)):
        return ops.gemm_partial_sums(x, weight)
    return linear(x, weight)
