"""The model: parts built from a plan, run in the plan's order.

One generic decoder serves every architecture; an architecture is its plan
(`liyab_amd.config.plan.ModelPlan`). The reference is built the same way:
one forward pass for all, steered by a registry row and a per-block plan
(docs/guide/architecture.md:47-55). Whole model, as the reference runs it
(src/core/transformer.cpp:6246-6258, 6284-6292): embedding (+ residual
position encoding) -> blocks in order -> final norm on the rows whose logits
are wanted -> head.
"""

from __future__ import annotations

from typing import Dict, List, Optional, Sequence, Tuple

import torch

from ..cache.pages import KVSpec, StateSpec
from ..kernels import ops
from ..config.plan import ModelPlan
from ..parts.base import StepContext
from ..parts.registry import build_part, find_part


class DecoderModel:
    def __init__(self, plan: ModelPlan, store, dtype: torch.dtype):
        self.plan = plan
        self.dtype = dtype
        self.width = plan.width
        self.vocab_size = plan.vocab_size
        self.max_positions = plan.max_positions
        self.embedding = build_part("embedding", plan.embedding, store, dtype)
        self.residual_position = (
            build_part("position", plan.residual_position, store, dtype) if plan.residual_position is not None else None
        )
        self.blocks = []
        for spec in plan.layers:
            mixer = build_part("mixer", spec.mixer, store, dtype)
            ffn = build_part("ffn", spec.ffn, store, dtype) if spec.ffn is not None else None
            norm_mixer = build_part("norm", spec.norm_mixer, store, dtype) if spec.norm_mixer is not None else None
            norm_ffn = build_part("norm", spec.norm_ffn, store, dtype) if spec.norm_ffn is not None else None
            self.blocks.append(find_part("block", spec.arrangement)(spec, mixer, ffn, norm_mixer, norm_ffn))
        self.final_norm = build_part("norm", plan.final_norm, store, dtype) if plan.final_norm is not None else None
        self.head = build_part("head", plan.head, store, dtype)
        self.order = list(plan.order)
        # the parts' step planners, one of each name (every attention layer shares attention's)
        self.step_planners = []
        for block in self.blocks:
            for part in (getattr(block, a, None) for a in ("mixer", "ffn", "norm_mixer", "norm_ffn")):
                planner = getattr(part, "step_planner", None)
                if planner is not None and all(p.name != planner.name for p in self.step_planners):
                    self.step_planners.append(planner)
        for e in self.order:
            if not (0 <= e.layer < len(self.blocks)) or not (0 <= e.cache_layer < len(self.blocks)):
                raise ValueError(f"the run order names layer {e.layer} / cache of {e.cache_layer}; the model has {len(self.blocks)}")

    # -- what the cache manager needs to know ---------------------------------
    def cache_groups(self) -> List[Tuple[KVSpec, List[int]]]:
        """Layers that own a cache, grouped by what they need of it."""
        owners = sorted({e.cache_layer for e in self.order})
        groups: Dict[tuple, Tuple[KVSpec, List[int]]] = {}
        for layer in owners:
            spec = self.blocks[layer].mixer.cache_spec()
            if spec is None:
                continue
            groups.setdefault(spec.key, (spec, []))[1].append(layer)
        return list(groups.values())

    def state_specs(self) -> Dict[int, StateSpec]:
        out = {}
        for layer in sorted({e.cache_layer for e in self.order}):
            spec = self.blocks[layer].mixer.state_spec()
            if spec is not None:
                out[layer] = spec
        return out

    # -- one step -----------------------------------------------------------
    def forward(self, ctx: StepContext, storage) -> Optional[torch.Tensor]:
        """Runs the step's tokens through every layer; returns float32 logits
        [n_logit_rows, vocab] or None when no row is wanted."""
        with ops.on_current_stream():
            return self._forward(ctx, storage)

    def _forward(self, ctx: StepContext, storage) -> Optional[torch.Tensor]:
        phases = ctx.phases
        if phases is not None:
            phases.mark("embed")
        x = ctx.workspace.get("residual", (ctx.n_tokens, self.width), torch.float32)
        fused = self.residual_position.fused_table() if self.residual_position is not None else None
        self.embedding.forward(ctx, x, position_table=fused)
        if self.residual_position is not None and fused is None:
            self.residual_position.add(ctx, x)
        pending = None  # the stream as a SplitStream while a layer has left it split (x is then stale)
        for e in self.order:
            block = self.blocks[e.layer]
            args = (x, ctx, storage.layer(e.cache_layer), storage.state(e.cache_layer))
            if getattr(block, "takes_pending", False):
                pending = block.forward(*args, writes_cache=e.writes_cache, pending=pending)
            else:
                if pending is not None:
                    pending.settle()
                    pending = None
                block.forward(*args, writes_cache=e.writes_cache)
        if phases is not None:
            phases.mark("lm_head")
            try:
                return self._head(ctx, x, pending)
            finally:
                phases.finish()
        return self._head(ctx, x, pending)

    def _head(self, ctx: StepContext, x, pending) -> Optional[torch.Tensor]:
        if ctx.n_logit_rows == 0:
            return None  # nobody reads the stream again
        if self.final_norm is not None:
            norm = self.final_norm
            kw = dict(rows=ctx.logit_rows, n_rows=ctx.n_logit_rows, name="head_in")
            rows = x
            if pending is not None:
                takes = getattr(norm, "takes_planes", None)
                rows = pending.planes if takes is not None and takes(pending.planes) else pending.settle()
            h = norm.lazy(rows, ctx, **kw) if hasattr(norm, "lazy") else norm.forward(rows, ctx, **kw)
        else:
            # no norm before the head: the wanted rows of the stream as they are, in the compute dtype
            rows = pending.settle() if pending is not None else x
            h = ctx.workspace.get("head_in", (ctx.n_logit_rows, self.width), self.dtype)
            ops.gather_rows(h, rows, ctx.logit_rows)
        return self.head.forward(h, ctx)
