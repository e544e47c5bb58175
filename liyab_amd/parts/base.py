"""What every part sees of a step, and the interfaces parts implement.

A step is a flat batch of tokens of several requests (the reference's
`Segment` list flattened: src/core/transformer.h:890-902, rows concatenated
in src/core/transformer.cpp:6689-6693). `StepContext` carries, per token,
its request and position, per request its block table and state slot, and
the rows whose logits are wanted. Parts read what they need from it; none
knows which model it is in or what else the batch holds.

Interfaces (duck-typed; the registries in `registry.py` map a spec's `kind`
to a class constructed as `cls(spec, store, dtype)`):

  norm:      forward(x_f32 [n, d], ctx, rows=None) -> [n or len(rows), d] in the compute dtype
  mixer:     cache_spec() -> KVSpec | None;  state_spec() -> StateSpec | None
             forward(h, ctx, cache, state, residual, writes_cache=True): adds its output into `residual`
  ffn:       forward(h, ctx, residual): adds its output into `residual`
  position:  where == "residual": add(ctx, x);  fused_table() -> table | None
  block:     cls(layer_spec, mixer, ffn, norm_mixer, norm_ffn); forward(x, ctx, cache, state, writes_cache)

A part that needs facts of a step laid out for its kernels (work lists, chunk tables), or whose
launches depend on more of the step than its sizes, has a class attribute `step_planner`: an
object with a `name` and `plan(facts: StepFacts) -> PartStepPlan`, called once a step for all
parts that share the name. Its words go to the device with the step's metadata, its key
becomes a term of the key under which the step's HIP graph is kept, and what its `make`
returns is handed to the parts as `ctx.plans[name]`. Attention's tiles are planned so
(`parts/attention.py`).

Optional, and only between parts that declare them: a mixer or feed-forward with `defers`
may be handed the stream as a `SplitStream` and may return one instead of adding in place;
a norm with `takes_planes` reads a split stream's planes; a block with `takes_pending` gets
and returns the split stream. A part without these sees plain tensors only.

`residual` is the float32 residual stream [n, d]; a part adds into it in
place (the sum is 32-bit whatever the compute dtype), which lets an output
projection fold the addition into its epilogue.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Callable, Dict, Hashable, List, Optional, Sequence, Tuple

import numpy as np
import torch


class SplitStream:
    """The residual stream as a sum of planes, float32 [parts, tokens, width]: its rows are
    planes[0] + planes[1] + ..., added in that order. A product cut over its inner dimension
    leaves the stream so: one plane of sums a part, the first of them also holding the bias
    and the stream the product was added to. `home` is the stream's own tensor [tokens,
    width], stale while the stream is split. Whoever reads the stream next adds the planes up
    as it loads its rows if it can (a norm with `takes_planes`, a product cut over its inner
    dimension in its turn); anything else gets `settle()`, which writes the sum to `home`."""

    def __init__(self, planes, home):
        self.planes, self.home = planes, home

    def settle(self):
        from ..kernels import ops

        ops.sum_parts(self.home, self.planes)
        return self.home


def settled(stream):
    """The residual stream as one tensor, its planes added up first if it is split."""
    return stream.settle() if isinstance(stream, SplitStream) else stream


class Workspace:
    """Named scratch buffers that keep their addresses from step to step."""

    def __init__(self, device):
        self.device = torch.device(device)
        self._bufs: Dict[tuple, torch.Tensor] = {}
        self._views: Dict[tuple, tuple] = {}  # the last view handed out under a name: (shape, tensor)
        self.generation = 0  # counts reallocations: captured graphs hold the old addresses

    def get(self, name: str, shape: Sequence[int], dtype: torch.dtype) -> torch.Tensor:
        key = (name, dtype)
        shape = tuple(shape)
        hit = self._views.get(key)
        if hit is not None and hit[0] == shape:
            return hit[1]  # the same view as last time: most calls of a decode loop
        n = 1
        for s in shape:
            n *= int(s)
        buf = self._bufs.get(key)
        if buf is None or buf.numel() < n:
            cap = max(n, 1)
            if buf is not None:
                cap = max(cap, 2 * buf.numel())
            buf = torch.empty(cap, dtype=dtype, device=self.device)
            self.generation += 1
            self._bufs[key] = buf
        view = buf[:n].view(*shape)
        self._views[key] = (shape, view)
        return view

    def bytes(self) -> int:
        return sum(b.numel() * b.element_size() for b in self._bufs.values())


class PhaseTimer:
    """Device time per phase of the model's forward pass (embed, each mixer kind, each
    feed-forward kind, lm_head), summed over steps: the reference's PhaseTimer adds wall time per
    phase the same way (src/core/transformer.cpp:463-481, phases in src/core/transformer.h:341-353)
    and its command line prints them per token (tools/liyab_cli.cpp:198-211). `mark(name)` says
    that the phase `name` starts now on the current stream; the time up to the next mark (or
    `finish`) is that phase's. Events are read only in `totals()`, which waits for the device.
    Steps are launched kernel by kernel while a timer is set: a replayed graph has no marks."""

    def __init__(self):
        self._marks = []  # (phase name or None for the end of a step, event)
        self._totals: Dict[str, float] = {}
        self.steps = 0

    def mark(self, name: Optional[str]) -> None:
        ev = torch.cuda.Event(enable_timing=True)
        ev.record()
        self._marks.append((name, ev))

    def finish(self) -> None:
        self.mark(None)
        self.steps += 1

    def totals(self) -> Dict[str, float]:
        """Milliseconds per phase since the timer was made (or `reset`)."""
        if self._marks:
            self._marks[-1][1].synchronize()
            for (name, ev), (_, nxt) in zip(self._marks, self._marks[1:]):
                if name is not None:
                    self._totals[name] = self._totals.get(name, 0.0) + ev.elapsed_time(nxt)
            self._marks = []
        return dict(self._totals)

    def reset(self) -> None:
        self._marks, self._totals, self.steps = [], {}, 0


@dataclass
class GroupStep:
    """A cache group's view of the step."""

    block_tables: torch.Tensor  # int32 [n_seqs, max_blocks]; -1 where unmapped
    slots: torch.Tensor  # int32 [n_tokens]: page * page_size + offset of each token


@dataclass
class StepHost:
    """The same facts on the host, for choosing kernels and grids."""

    q_lens: List[int]  # tokens of each request in this step
    starts: List[int]  # row of each request's first token
    first_pos: List[int]  # position of each request's first token
    max_q_len: int
    max_context: int  # longest context after this step


@dataclass
class StepFacts:
    """What a part's step planner sees of a step, on the host, before anything is launched."""

    n_tokens: int
    n_seqs: int
    q_lens: np.ndarray  # intc [n_seqs]: tokens each request brings
    first_pos: np.ndarray  # intc [n_seqs]: each request's length before the step
    state_slots: np.ndarray  # intc [n_seqs]
    max_q_len: int
    max_context: int
    page_size: int


@dataclass
class PartStepPlan:
    """What a part's planner decides for one step.

    `key`: everything the part's launches (kernels chosen, grids, scalar arguments) depend on
    besides the step's sizes (tokens, requests, wanted rows); two steps with equal sizes and
    equal keys of all planners replay one captured graph, so whatever else varies must reach
    the kernels through `words`. `n_words` int32 words go to the device behind the step's
    common metadata in the same copy; `fill(address)` writes them into pinned host memory
    (a `ctypes` pointer to int32); their count must be a function of the key. `make(words)`
    (words: the int32 device tensor of n_words, or None) returns what parts find in
    `ctx.plans[name]`. `recurs`: whether a step of this kind tends to come back the same
    (decode steps do; a mix of prompt portions mostly does not, and is captured later)."""

    key: Hashable
    n_words: int = 0
    fill: Optional[Callable[[Any], None]] = None
    make: Optional[Callable[[Optional[torch.Tensor]], Any]] = None
    recurs: bool = True


@dataclass
class StepContext:
    n_tokens: int
    n_seqs: int
    token_ids: torch.Tensor  # int32 [n_tokens]
    positions: torch.Tensor  # int32 [n_tokens]
    tok_seq: torch.Tensor  # int32 [n_tokens]: index of the token's request in this step
    seq_starts: torch.Tensor  # int32 [n_seqs + 1]
    context_lens: torch.Tensor  # int32 [n_seqs]: positions each request holds after this step
    state_slots: torch.Tensor  # int32 [n_seqs]
    logit_rows: torch.Tensor  # int32 [n_rows]
    n_logit_rows: int
    groups: List[GroupStep]
    host: StepHost
    workspace: Workspace
    dtype: torch.dtype
    page_size: int
    logit_slots: Optional[torch.Tensor] = None  # int32 [n_rows]: state slot of each wanted row's request
    last_tokens: Optional[torch.Tensor] = None  # int32 [slots]: the token each request drew last (on the device)
    plans: Dict[str, Any] = field(default_factory=dict)  # what each part's step planner made for this step, by its name
    phases: Optional[PhaseTimer] = None  # set: the model and its blocks mark where each phase starts
