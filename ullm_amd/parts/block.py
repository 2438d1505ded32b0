"""Pre-norm residual block: h += mixer(norm1(h)); h += ffn(norm2(h)).

The reference carries (branch output, residual) between layers and lets the next norm do the add
(ullm/models/qwen3.py:159-178, ullm/layers/layernorm.py:24-26).  The same trick is kept: a branch
output is left ``pending`` and added inside the next fused add+norm kernel, which saves one pass
over the residual stream per branch.
"""
from __future__ import annotations

from .base import Block, FeedForward, LayerCache, Mixer, Norm, StepContext, register_part


@register_part("block", "prenorm")
class PreNormBlock(Block):
    def __init__(self, mixer_norm: Norm, mixer: Mixer, ffn_norm: Norm, ffn: FeedForward):
        self.mixer_norm, self.mixer, self.ffn_norm, self.ffn = mixer_norm, mixer, ffn_norm, ffn

    def children(self):
        return [self.mixer_norm, self.mixer, self.ffn_norm, self.ffn]

    def cache_need(self):
        return self.mixer.cache_need()

    def forward(self, residual, pending, ctx: StepContext, cache: LayerCache):
        # Each half: the norm kernel adds the pending branch into the stream and normalises; the
        # part then either adds its result into the stream itself (folded into its last kernel,
        # where it offers that for this batch) or returns it as the next pending branch.
        # Where nothing is left to add, a part that folds the norm into its first projection gets
        # the norm as a record instead of its result: then a half is two or three kernels.
        if self.mixer.fusable(residual, ctx):
            self.mixer.forward_fused(self._normed(self.mixer_norm, self.mixer, pending, residual, ctx), residual, ctx,
                                     cache)
            pending = None
        else:
            pending = self.mixer.forward(self.mixer_norm.add_norm(pending, residual, out_dtype=ctx.dtype), ctx, cache)
        if self.ffn.fusable(residual, ctx):
            self.ffn.forward_fused(self._normed(self.ffn_norm, self.ffn, pending, residual, ctx), residual, ctx)
            return residual, None
        return residual, self.ffn.forward(self.ffn_norm.add_norm(pending, residual, out_dtype=ctx.dtype), ctx)

    @staticmethod
    def _normed(norm: Norm, part, pending, residual, ctx: StepContext):
        if pending is None and part.folds_norm:
            record = norm.pending(residual, ctx.dtype)
            if record is not None:
                return record
        return norm.add_norm(pending, residual, out_dtype=ctx.dtype)
