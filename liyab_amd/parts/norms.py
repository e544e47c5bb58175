"""Norm parts."""

from __future__ import annotations

from typing import Optional

import torch

from ..kernels import ops
from .base import StepContext
from .registry import register_norm


class LayerNorm:
    """y = (x - mean) / sqrt(var + eps) * weight + bias over the last axis
    (the reference's layernorm, src/core/transformer.cpp:77-106); weight and
    bias are each optional, as there (:1105-1109). Statistics are 32-bit."""

    def __init__(self, spec, store, dtype: torch.dtype):
        self.width = spec.width
        self.eps = float(spec.eps)
        self.dtype = dtype
        w = spec.tensors.get("weight")
        b = spec.tensors.get("bias")
        self.weight = store.fetch(w, (self.width,), "vector") if w is not None else None
        self.bias = store.fetch(b, (self.width,), "vector") if b is not None else None

    def forward(self, x: torch.Tensor, ctx: StepContext, rows: Optional[torch.Tensor] = None,
                n_rows: Optional[int] = None, name: str = "normed") -> torch.Tensor:
        n = x.shape[0] if rows is None else (n_rows if n_rows is not None else rows.numel())
        out = ctx.workspace.get(name, (n, self.width), self.dtype)
        ops.layernorm(out, x, self.weight, self.bias, self.eps, rows=rows)
        return out


register_norm("layernorm", LayerNorm)
