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

    def forward(self, x: torch.Tensor, ctx: StepContext, cache, state, writes_cache: bool = True) -> None:
        h = self.norm_mixer.forward(x, ctx)
        self.mixer.forward(h, ctx, cache, state, x, writes_cache=writes_cache)
        if self.ffn is not None:
            h = self.norm_ffn.forward(x, ctx)
            self.ffn.forward(h, ctx, x)


register_block("pre_norm", PreNormBlock)
