"""Pre-norm residual block: h += mixer(norm1(h)); h += ffn(norm2(h)).

The reference carries (branch output, residual) between layers and lets the next norm do the add
(ullm/models/qwen3.py:159-178, ullm/layers/layernorm.py:24-26).  The same trick is kept: a branch
output is left ``pending`` and added inside the next fused add+norm kernel, which saves one pass
over the residual stream per branch.
"""
from __future__ import annotations

from typing import Optional

from .base import Block, FeedForward, LayerCache, Mixer, Norm, PendingNorm, StepContext, register_part


@register_part("block", "prenorm")
class PreNormBlock(Block):
    hands_norm_ahead = True

    def __init__(self, mixer_norm: Norm, mixer: Mixer, ffn_norm: Norm, ffn: FeedForward):
        self.mixer_norm, self.mixer, self.ffn_norm, self.ffn = mixer_norm, mixer, ffn_norm, ffn

    def children(self):
        return [self.mixer_norm, self.mixer, self.ffn_norm, self.ffn]

    def cache_need(self):
        return self.mixer.cache_need()

    def entry_norm(self):
        return self.mixer_norm

    def forward(self, residual, pending, ctx: StepContext, cache: LayerCache, next_norm: Optional[Norm] = None):
        # Each half: the norm kernel adds the pending branch into the stream and normalises; the
        # part then either adds its result into the stream itself (folded into its last kernel,
        # where it offers that for this batch) or returns it as the next pending branch.
        # Where nothing is left to add, a part that folds the norm into its first projection gets
        # the norm as a record instead of its result: then a half is two or three kernels.  A part
        # whose last kernel can also prepare the norm that follows is told which one that is, and
        # what it returns is the record for the part behind that norm.
        if self.mixer.fusable(residual, ctx):
            x = self._normed(self.mixer_norm, self.mixer, pending, residual, ctx)
            if self.mixer.hands_norm_ahead:
                pending = self.mixer.forward_fused(x, residual, ctx, cache, then=self.ffn_norm)
            else:
                pending = self.mixer.forward_fused(x, residual, ctx, cache)
        else:
            pending = self.mixer.forward(self._normed(self.mixer_norm, None, pending, residual, ctx), ctx, cache)
        if self.ffn.fusable(residual, ctx):
            x = self._normed(self.ffn_norm, self.ffn, pending, residual, ctx)
            if self.ffn.hands_norm_ahead:
                return residual, self.ffn.forward_fused(x, residual, ctx, then=next_norm)
            return residual, self.ffn.forward_fused(x, residual, ctx)
        return residual, self.ffn.forward(self._normed(self.ffn_norm, None, pending, residual, ctx), ctx)

    @staticmethod
    def _normed(norm: Norm, part, pending, residual, ctx: StepContext):
        """The input of the part behind ``norm``: the normed stream, or the norm as a record where nothing is
        left to add and ``part`` (None: a part that wants its input computed) folds it into its first product."""
        if isinstance(pending, PendingNorm):
            # the stream is complete and a product has prepared a norm: this one, by the way it was asked for
            if part is not None and part.folds_norm and pending.norm is norm:
                return pending
            pending = None
        if pending is None and part is not None and part.folds_norm:
            record = norm.pending(residual, ctx.dtype)
            if record is not None:
                return record
        return norm.add_norm(pending, residual, out_dtype=ctx.dtype)
