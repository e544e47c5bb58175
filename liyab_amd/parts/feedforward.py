"""Feed-forward parts."""

from __future__ import annotations

import torch

from .base import StepContext, settled
from .linear import linear, linear_deferred
from .registry import register_ffn


class DenseFFN:
    """The ungated feed-forward: m = act(h . Wup^T + b_up) . Wdown^T + b_down,
    added into the residual (the reference's dense_ffn for FfnKind::Ungated,
    src/core/transformer.cpp:4903-4913; residual :5692). `activation` is
    "gelu_tanh" (:123-130) or "gelu_erf" (:134-142)."""

    # every launch goes through the kernel library and depends on nothing of this object but its
    # tensors and the constants among its attributes: layers of this kind may run from one recorded list
    replayable = True
    # rows behind the step's tokens (token 0 at position 0 of the first request, slot -1) are computed
    # and never read: nothing here writes for them or lets them touch another row
    takes_padding_rows = True

    def __init__(self, spec, store, dtype: torch.dtype):
        self.dtype = dtype
        self.width, self.inner, self.activation = spec.width, spec.inner, spec.activation
        if self.activation not in ("gelu_tanh", "gelu_erf"):
            raise ValueError(f"unknown activation '{self.activation}'")
        t = spec.tensors
        self.up_weight = store.fetch(t["up_weight"], (self.inner, self.width), "matrix")
        self.up_bias = store.fetch(t["up_bias"], (self.inner,), "vector") if "up_bias" in t else None
        self.down_weight = store.fetch(t["down_weight"], (self.width, self.inner), "matrix")
        self.down_bias = store.fetch(t["down_bias"], (self.width,), "vector") if "down_bias" in t else None

    defers = True  # forward(..., defer=True) takes the stream split or whole and may hand it back split

    def forward(self, h, ctx: StepContext, residual: torch.Tensor, defer: bool = False):
        """Adds the feed-forward's output into `residual`. With `defer`, `residual` may be a
        SplitStream, and where the second product runs faster cut over its inner dimension the
        stream with the output added comes back as a SplitStream (None: added in place, to
        the stream's own tensor)."""
        inner = ctx.workspace.get("ffn_inner", (h.shape[0], self.inner), self.dtype)
        linear(h, self.up_weight, self.up_bias, out=inner, activation=self.activation)
        split = linear_deferred(inner, self.down_weight, self.down_bias, ctx, "ffn_parts", residual) if defer else None
        if split is None:
            linear(inner, self.down_weight, self.down_bias, residual=settled(residual))
        return split


register_ffn("dense_ffn", DenseFFN)
