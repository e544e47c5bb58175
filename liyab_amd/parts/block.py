"""How a layer's parts are arranged."""

from __future__ import annotations

import torch

from .base import SplitStream, StepContext, settled
from .registry import register_block


class PreNormBlock:
    """x += mixer(norm_mixer(x)); x += ffn(norm_ffn(x)): the reference's
    run_block for a sequential pre-norm layer (src/core/transformer.cpp:5514-5726:
    norm :5565-5577, mixer, residual :5647, norm :5663-5666, ffn, residual :5692)."""

    # every launch goes through the kernel library and depends on nothing of this object but its
    # tensors and the constants among its attributes: layers of this kind may run from one recorded list
    replayable = True
    # rows behind the step's tokens (token 0 at position 0 of the first request, slot -1) are computed
    # and never read: nothing here writes for them or lets them touch another row
    takes_padding_rows = True

    def __init__(self, spec, mixer, ffn, norm_mixer, norm_ffn):
        self.mixer, self.ffn, self.norm_mixer, self.norm_ffn = mixer, ffn, norm_mixer, norm_ffn
        # phases are named after the parts' kinds (the reference's: attention, dense_ffn, ...)
        self.mixer_phase = getattr(getattr(spec, "mixer", None), "kind", "mixer")
        self.ffn_phase = getattr(getattr(spec, "ffn", None), "kind", "ffn")

    takes_pending = True  # forward(..., pending=) takes the stream split and may return it split

    def forward(self, x: torch.Tensor, ctx: StepContext, cache, state, writes_cache: bool = True, pending=None):
        """x: the residual stream's own tensor. `pending`: the stream as a SplitStream when the
        previous layer left it split (x is then stale). Returns the stream as a SplitStream if
        this layer leaves it split, else None (x holds it)."""
        stream = pending if pending is not None else x
        if ctx.phases is not None:
            ctx.phases.mark(self.mixer_phase)
        h, stream = self._normed(self.norm_mixer, stream, ctx)
        if getattr(self.mixer, "defers", False):
            stream = self.mixer.forward(h, ctx, cache, state, stream, writes_cache=writes_cache, defer=True) or x
        else:
            self.mixer.forward(h, ctx, cache, state, settled(stream), writes_cache=writes_cache)
            stream = x
        if self.ffn is not None:
            if ctx.phases is not None:
                ctx.phases.mark(self.ffn_phase)
            h, stream = self._normed(self.norm_ffn, stream, ctx)
            if getattr(self.ffn, "defers", False):
                stream = self.ffn.forward(h, ctx, stream, defer=True) or x
            else:
                self.ffn.forward(h, ctx, settled(stream))
                stream = x
        return stream if isinstance(stream, SplitStream) else None

    @staticmethod
    def _normed(norm, stream, ctx):
        """The norm of the stream and the stream as it is afterwards (settled if the norm cannot
        read it split). The norm's output is left pending when the norm allows it, so that the
        next product may fold it in (parts that need the rows call `as_tensor`)."""
        rows = stream
        if isinstance(stream, SplitStream):
            takes = getattr(norm, "takes_planes", None)
            if takes is not None and takes(stream.planes):
                rows = stream.planes
            else:
                rows = stream = stream.settle()
        return (norm.lazy(rows, ctx) if hasattr(norm, "lazy") else norm.forward(rows, ctx)), stream


register_block("pre_norm", PreNormBlock)
