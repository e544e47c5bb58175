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

import bisect
import dataclasses
import os

import numpy as np

from ..cache.pages import KVSpec, StateSpec
from ..kernels import lib as _lib
from ..kernels import ops
from ..config.plan import ModelPlan
from ..parts.base import SplitStream, StepContext
from ..parts.registry import build_part, find_part


_OTHER = object()  # stands for "holds something that may not be run from a recorded list"


def _describe(obj, tensors: list, seen: set):
    """What a part is made of, as a hashable key, its tensors appended to `tensors` in the order
    they are met: two layers with equal keys hold tensors of equal shapes in the same places
    and equal constants everywhere else. _OTHER if something in it is not `replayable`."""
    if isinstance(obj, torch.Tensor):
        tensors.append(obj)
        return ("tensor", tuple(obj.shape), str(obj.dtype), tuple(obj.stride()))
    if obj is None or isinstance(obj, (bool, int, float, str)):
        return obj
    if isinstance(obj, torch.dtype):
        return str(obj)
    if isinstance(obj, (list, tuple)):
        items = tuple(_describe(v, tensors, seen) for v in obj)
        return _OTHER if any(i is _OTHER for i in items) else ("seq", items)
    if isinstance(obj, dict):
        items = tuple((str(k), _describe(v, tensors, seen)) for k, v in sorted(obj.items(), key=lambda kv: str(kv[0])))
        return _OTHER if any(i is _OTHER for _, i in items) else ("dict", items)
    if dataclasses.is_dataclass(obj) and not isinstance(obj, type):
        # a spec the part was built from: it names this layer's tensors; what the part computes with
        # it has copied into attributes of its own
        return ("spec", type(obj).__name__)
    if not getattr(type(obj), "replayable", False) or id(obj) in seen or not hasattr(obj, "__dict__"):
        return _OTHER
    seen.add(id(obj))
    fields = []
    for name in sorted(vars(obj)):
        key = _describe(vars(obj)[name], tensors, seen)
        if key is _OTHER:
            return _OTHER
        fields.append((name, key))
    return (type(obj).__module__, type(obj).__qualname__, tuple(fields))


class _Recorded:
    """A layer's launches as a list of words, and where in it the addresses of the layer's own
    tensors stand (any address inside one of them, as an offset from its start). `addresses`: which
    words are addresses at all; a size or a constant that happens to lie in a tensor's range is not one."""

    def __init__(self, words: np.ndarray, addresses: np.ndarray, bases: np.ndarray, sizes, pending_out):
        self.words = words
        self.pending_out = pending_out
        order = np.argsort(bases)
        starts = bases[order].tolist()
        positions, which, offsets = [], [], []
        self.usable = True
        for i in range(1, len(starts)):
            if starts[i] < starts[i - 1] + sizes[order[i - 1]]:
                self.usable = False  # two of the layer's tensors overlap: an address would name both
        listed = words.tolist()
        for at in np.flatnonzero(addresses).tolist():
            word = listed[at]
            j = bisect.bisect_right(starts, word) - 1
            if j >= 0 and word < starts[j] + sizes[order[j]]:
                positions.append(at)
                which.append(int(order[j]))
                offsets.append(word - starts[j])
        self.positions = np.array(positions, dtype=np.int64)
        self.which = np.array(which, dtype=np.int64)
        self.offsets = np.array(offsets, dtype=np.uint64)

    def for_layer(self, bases: np.ndarray) -> np.ndarray:
        words = self.words.copy()
        words[self.positions] = bases[self.which] + self.offsets
        return words


class _NoRecording:
    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


_no_recording = _NoRecording()


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
        # Layers of one kind run from one recorded list of launches (csrc/replay.hip): a layer's kind
        # is what its block and parts are made of, its tensors aside; layers whose parts are not all
        # `replayable` run through their Python every time. LIYAB_REPLAY=0 switches it off.
        self.replay_layers = os.environ.get("LIYAB_REPLAY", "1") != "0"
        self._layer_kind, self._layer_tensors = [], []
        for block in self.blocks:
            tensors: list = []
            self._layer_kind.append(_describe(block, tensors, set()))
            self._layer_tensors.append(tensors)
        self.replayed_layers = 0  # layers that ran from a recorded list, over the model's lifetime
        # A step may carry padding rows behind its tokens (engine/step.py: padded_rows) when every part that
        # sees all the step's rows says that it takes them (`takes_padding_rows`): the embedding, a position
        # encoding of the stream, and every block with its mixer, feed-forward and norms. The final norm and
        # the head see the wanted rows only.
        every = [self.embedding, self.residual_position]
        for block in self.blocks:
            every += [block] + [getattr(block, a, None) for a in ("mixer", "ffn", "norm_mixer", "norm_ffn")]
        self.takes_padding_rows = all(bool(getattr(part, "takes_padding_rows", False)) for part in every if part is not None)

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
        recorded = {}  # this step's lists of launches, by the kind of layer and the state it found the stream in
        for e in self.order:
            block = self.blocks[e.layer]
            cache, state = storage.layer(e.cache_layer), storage.state(e.cache_layer)
            key = None
            if self.replay_layers and phases is None and self._layer_kind[e.layer] is not _OTHER:
                own = self._layer_tensors[e.layer] + (list(cache.rows.values()) if cache is not None else []) + ([state] if state is not None else [])
                key = (self._layer_kind[e.layer], cache.group if cache is not None else -1,
                       tuple((tuple(t.shape), str(t.dtype)) for t in own[len(self._layer_tensors[e.layer]):]), e.writes_cache,
                       None if pending is None else (pending.planes.data_ptr(), tuple(pending.planes.shape)))
                bases = np.fromiter((t.data_ptr() for t in own), dtype=np.uint64, count=len(own))
                hit = recorded.get(key)
                if hit is not None and hit.usable:
                    _lib.replay(hit.for_layer(bases))
                    pending = hit.pending_out
                    self.replayed_layers += 1
                    continue
            args = (x, ctx, cache, state)
            with _lib.recording() if key is not None and key not in recorded else _no_recording as rec:
                if getattr(block, "takes_pending", False):
                    pending = block.forward(*args, writes_cache=e.writes_cache, pending=pending)
                else:
                    if pending is not None:
                        pending.settle()
                        pending = None
                    block.forward(*args, writes_cache=e.writes_cache)
            if rec is not None and rec.words is not None and (pending is None or isinstance(pending, SplitStream)):
                recorded[key] = _Recorded(rec.words, rec.addresses, bases, [t.numel() * t.element_size() for t in own], pending)
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
