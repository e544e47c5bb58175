"""The output head."""

from __future__ import annotations

import torch

from ..kernels import ops
from .base import StepContext
from .linear import linear
from .registry import register_head


class LMHead:
    """logits = h . W^T (+ bias), times logit_scale when it is not 1: the
    reference's compute_logits after the final norm (src/core/transformer.cpp:2622-2638,
    finish_logits :2613-2620). W may be the token embedding's table (a tied
    head, :1100-1104): the store hands out the same device tensor for the same
    name, so a tied table is resident once. Logits are float32."""

    def __init__(self, spec, store, dtype: torch.dtype):
        self.width, self.vocab_size = spec.width, spec.vocab_size
        self.logit_scale = float(spec.logit_scale)
        t = spec.tensors
        self.weight = store.fetch(t["weight"], (self.vocab_size, self.width), "table")
        self.bias = store.fetch(t["bias"], (self.vocab_size,), "vector") if "bias" in t else None

    def forward(self, h, ctx: StepContext) -> torch.Tensor:
        logits = ctx.workspace.get("logits", (h.shape[0], self.vocab_size), torch.float32)
        linear(h, self.weight, self.bias, out=logits)
        if self.logit_scale != 1.0:
            ops.scale_(logits, self.logit_scale)  # after the bias, as the reference's finish_logits does (:2613-2620)
        return logits


register_head("lm_head", LMHead)
