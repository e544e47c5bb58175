"""How a layer's parts are arranged."""

from __future__ import annotations

import torch

from .base import StepContext
from .registry import register_block


class PreNormBlock:
    """x += mixer(norm_mixer(x)); x += ffn(norm_ffn(x)): the reference's
    run_block for a sequential pre-norm layer (src/core/transformer.cpp:5514-5726:
    norm :5565-5577, mixer, residual :5647, norm :5663-5666, ffn, residual :5692)."""

    def __init__(self, spec, mixer, ffn, norm_mixer, norm_ffn):
        self.mixer, self.ffn, self.norm_mixer, self.norm_ffn = mixer, ffn, norm_mixer, norm_ffn

    takes_pending = True  # forward(..., pending=) takes sums the stream still lacks and may return such

    def forward(self, x: torch.Tensor, ctx: StepContext, cache, state, writes_cache: bool = True, pending=None):
        """`pending`: PendingSums that x still lacks (the previous layer's), added by this
        layer's first norm as it reads x. Returns this layer's own, or None."""
        if pending is not None and getattr(self.norm_mixer, "takes_sums", False):
            h = self.norm_mixer.forward(x, ctx, sums=pending.sums)
        else:
            if pending is not None:
                pending.settle(x)
            h = self._normed(self.norm_mixer, x, ctx)
        pending = None
        if getattr(self.mixer, "defers", False):
            pending = self.mixer.forward(h, ctx, cache, state, x, writes_cache=writes_cache, defer=True)
        else:
            self.mixer.forward(h, ctx, cache, state, x, writes_cache=writes_cache)
        if self.ffn is None:
            return pending
        if pending is not None and getattr(self.norm_ffn, "takes_sums", False):
            h = self.norm_ffn.forward(x, ctx, sums=pending.sums)
        else:
            if pending is not None:
                pending.settle(x)
            h = self._normed(self.norm_ffn, x, ctx)
        if getattr(self.ffn, "defers", False):
            return self.ffn.forward(h, ctx, x, defer=True)
        self.ffn.forward(h, ctx, x)
        return None

    @staticmethod
    def _normed(norm, x, ctx):
        """The norm's output, left pending when the norm allows it so that the next product
        may fold it in (parts that need the rows call `as_tensor`)."""
        return norm.lazy(x, ctx) if hasattr(norm, "lazy") else norm.forward(x, ctx)


register_block("pre_norm", PreNormBlock)
