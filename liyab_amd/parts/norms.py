"""Norm parts."""

from __future__ import annotations

from typing import Optional

import torch

from ..kernels import ops
from .base import StepContext
from .registry import register_norm


class Normed:
    """A norm's output that has not been computed yet: what a block hands to its mixer or
    feed-forward. A product kernel that can apply the norm to its own first operand takes
    it as it is (`linear` does); anything else calls `tensor()` and gets the rows."""

    def __init__(self, norm, x: torch.Tensor, ctx: StepContext, rows=None, n_rows=None, name="normed"):
        self.norm, self.x, self.ctx, self.rows, self.name = norm, x, ctx, rows, name
        # x: the rows [n, d], or a sum of planes [parts, n, d] for a norm that `takes_planes`
        self.n_rows = x.shape[-2] if rows is None else (n_rows if n_rows is not None else rows.numel())
        self._tensor = None

    @property
    def shape(self):
        return (self.n_rows, self.norm.width)

    @property
    def dtype(self):
        return self.norm.dtype

    def tensor(self) -> torch.Tensor:
        if self._tensor is None:
            self._tensor = self.norm.forward(self.x, self.ctx, rows=self.rows, n_rows=self.n_rows, name=self.name)
        return self._tensor


def as_tensor(h) -> torch.Tensor:
    """The rows of a part's input, computing a pending norm if there is one."""
    return h.tensor() if isinstance(h, Normed) else h


class LayerNorm:
    """y = (x - mean) / sqrt(var + eps) * weight + bias over the last axis
    (the reference's layernorm, src/core/transformer.cpp:77-106); weight and
    bias are each optional, as there (:1105-1109). Statistics are 32-bit."""

    # every launch goes through the kernel library and depends on nothing of this object but its
    # tensors and the constants among its attributes: layers of this kind may run from one recorded list
    replayable = True
    # rows behind the step's tokens (token 0 at position 0 of the first request, slot -1) are computed
    # and never read: nothing here writes for them or lets them touch another row
    takes_padding_rows = True

    def __init__(self, spec, store, dtype: torch.dtype):
        self.width = spec.width
        self.eps = float(spec.eps)
        self.dtype = dtype
        w = spec.tensors.get("weight")
        b = spec.tensors.get("bias")
        self.weight = store.fetch(w, (self.width,), "vector") if w is not None else None
        self.bias = store.fetch(b, (self.width,), "vector") if b is not None else None

    fusable = "layernorm"  # product kernels know how to fold this norm into their operand

    def takes_planes(self, planes: torch.Tensor) -> bool:
        """Whether forward() and lazy() take these planes [parts, n, d] of a split residual stream
        in place of rows, adding them up as the rows are loaded."""
        return ops.norm_takes_planes(self.width)

    def lazy(self, x: torch.Tensor, ctx: StepContext, rows: Optional[torch.Tensor] = None,
             n_rows: Optional[int] = None, name: str = "normed") -> Normed:
        return Normed(self, x, ctx, rows, n_rows, name)

    def forward(self, x: torch.Tensor, ctx: StepContext, rows: Optional[torch.Tensor] = None,
                n_rows: Optional[int] = None, name: str = "normed") -> torch.Tensor:
        n = x.shape[-2] if rows is None else (n_rows if n_rows is not None else rows.numel())
        out = ctx.workspace.get(name, (n, self.width), self.dtype)
        ops.layernorm(out, x, self.weight, self.bias, self.eps, rows=rows)
        return out


register_norm("layernorm", LayerNorm)
