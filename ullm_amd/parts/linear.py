"""y = x W^T (+ b) with W stored [out, in] as the reference's linears are
(ullm/layers/linear.py:165,268).  The float32 mode always takes the hand-written 32-bit kernel
(fixed K order, no matrix-core input rounding); bfloat16 takes the skinny weight-streaming kernel
for few rows and the library product for many, as the reference uses a library product throughout.
"""
from __future__ import annotations

from typing import Optional

import torch

from ..kernels import dispatch, ops


def linear(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None,
           out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    out_dtype = out_dtype or x.dtype
    if x.dtype == torch.float32 or weight.dtype == torch.float32:
        return ops.gemm_simple(x, weight, bias, out_dtype=out_dtype)
    return ops.gemm_bf16(x, weight, bias, out_dtype=out_dtype)


def linear_of_norm(x, weight: torch.Tensor, bias: Optional[torch.Tensor] = None, silu: bool = False) -> torch.Tensor:
    """The first projection of a part whose input may be a norm not yet computed
    (:class:`~ullm_amd.parts.base.PendingNorm`): then the norm is folded into the product where the
    kernel takes the shapes, and computed first where not.  With ``silu`` the weights are gate | up
    and the result silu(gate) * up."""
    from .base import PendingNorm
    if isinstance(x, PendingNorm) and x.scaled is not None:
        y = _linear_of_prepared_norm(x, weight, bias, silu)
        if y is not None:
            return y
    if isinstance(x, PendingNorm):
        # folding the norm into the product pays up to a row count that depends on the matrix: beyond, the 32-bit
        # rows of X cost every block more registers and loads than the saved launch is worth
        if (x.out_dtype == torch.bfloat16
                and x.stream.shape[0] <= dispatch.limits(weight.shape[0], weight.shape[1]).fold_norm
                and ops.gemm_skinny_normed_supports(x.stream, x.gain, weight)):
            return ops.gemm_skinny_normed(x.stream, x.gain, x.eps, weight, bias, silu=silu)
        x = x.apply()
    if silu:
        return gate_up(x, weight)
    return linear(x, weight, bias)


def _linear_of_prepared_norm(x, weight: torch.Tensor, bias: Optional[torch.Tensor], silu: bool) -> Optional[torch.Tensor]:
    """The product of a norm that the product before prepared (``x.scaled`` = stream * gain, ``x.squares``): the
    kernel the matrix's limits name for this row count multiplies ``x.scaled`` and scales its rows.  None where no
    kernel takes the shapes."""
    a, rows = x.scaled, x.scaled.shape[0]
    if a.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16 or rows > ops.NORMED_MAX_ROWS:
        return None
    lim = dispatch.limits(weight.shape[0], weight.shape[1])
    few = ops.gemm_skinny_supports(a, weight)
    if silu:
        if few and rows <= lim.silu_skinny:
            return ops.gemm_skinny_silu(a, weight, squares=x.squares, eps=x.eps)
        if ops.gemm_rows_supports(a, weight, silu=True):
            return ops.gemm_rows(a, weight, silu=True, squares=x.squares, eps=x.eps)
        return ops.gemm_skinny_silu(a, weight, squares=x.squares, eps=x.eps) if few else None
    if few and rows <= lim.skinny:
        return ops.gemm_skinny(a, weight, bias, squares=x.squares, eps=x.eps)
    if ops.gemm_rows_supports(a, weight):
        return ops.gemm_rows(a, weight, bias, squares=x.squares, eps=x.eps)
    return ops.gemm_skinny(a, weight, bias, squares=x.squares, eps=x.eps) if few else None


def add_into_stream(x: torch.Tensor, weight: torch.Tensor, residual: torch.Tensor, then=None,
                    out_dtype: Optional[torch.dtype] = None):
    """residual += x W^T by the few-rows kernel (the caller has asked :func:`can_fuse`).  With ``then``, the norm
    that is applied to the stream next, the same kernel also prepares that norm where it can (the stream times
    the norm's gain, the rows' sums of squares) and the result is the norm's record for the part behind it;
    otherwise None."""
    gain = then.ahead_gain() if then is not None else None
    if (gain is not None and residual.shape[0] <= ops.NORMED_MAX_ROWS and weight.shape[0] % 4 == 0
            and gain.dtype == torch.float32 and gain.numel() == weight.shape[0] and gain.data_ptr() % 16 == 0):
        scaled, squares = ops.gemm_skinny_add(x, weight, residual, next_gain=gain)
        return then.pending(residual, out_dtype or x.dtype, scaled, squares)
    ops.gemm_skinny_add(x, weight, residual)
    return None


def gate_up(x: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
    """silu(x g^T) * (x u^T) for the stacked weights g | u [2 I, K]: by the few-rows kernel or the kernel for up
    to 128 rows with the activation on store, up to the row counts the matrix's limits name; else by the
    library product and the activation kernel (float32 always: the 32-bit product, then the kernel)."""
    rows = x.shape[0]
    if x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16:
        lim = dispatch.limits(weight.shape[0], weight.shape[1])
        if rows <= lim.silu_skinny and ops.gemm_skinny_supports(x, weight):
            return ops.gemm_skinny_silu(x, weight)
        if rows <= min(lim.silu_rows, ops.ROWS_MAX_ROWS) and ops.gemm_rows_supports(x, weight, silu=True):
            return ops.gemm_rows(x, weight, silu=True)
    return ops.silu_mul(linear(x, weight))


FUSED_MAX_ROWS = 16      # the few-rows kernel adds into the stream itself for up to this many rows (one tile of X)


def can_fuse(residual: torch.Tensor, dtype: torch.dtype, *weights: torch.Tensor) -> bool:
    """True if the folded projection kernels take this batch: bfloat16 compute, few rows, row lengths
    that keep 16-byte alignment."""
    T, H = residual.shape
    if dtype != torch.bfloat16 or T > FUSED_MAX_ROWS or H % 8:
        return False
    return all(w.dtype == torch.bfloat16 and w.shape[1] % 8 == 0 and w.shape[0] % 4 == 0 and w.data_ptr() % 16 == 0
               for w in weights)


def linear_into_stream(x: torch.Tensor, weight: torch.Tensor, ctx) -> torch.Tensor:
    """The last projection of a mixer or feed-forward, whose result the next norm adds to the residual
    stream.  For a range of row counts that depends on the matrix (17 to 256 for all but small ones), in
    bfloat16 and where the model's norms add stacks, it is a stack of float32 partial sums over slices of
    the inner dimension (the slices fill the chip, the norm adds them in order); otherwise the plain
    product.  For few long rows the library's choice of kernel is two to five times off the memory
    roofline at these row counts."""
    lim = dispatch.limits(weight.shape[0], weight.shape[1])
    if (ctx.stacked_branches and x.dtype == torch.bfloat16 and lim.stacked_from > 0
            and lim.stacked_from <= x.shape[0] <= lim.stacked_to and ops.gemm_partial_sums_supports(x, weight)):
        return ops.gemm_partial_sums(x, weight)
    return linear(x, weight)
