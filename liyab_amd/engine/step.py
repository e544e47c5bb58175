"""The step function: one batch of (request, its next tokens) through the model.

The counterpart of the reference's `Transformer::forward_batch`
(src/core/transformer.cpp:6589-6769): items of many tokens (a portion of a
prompt, continuing where the request's cache ends) beside items of one token
(decoding), each of a different request (:6607-6647); rows are the items
concatenated, a row's position is its request's length plus its index in
the item (:6689-6697); every block runs over all rows at once and only
attention looks at a row's own request; logits are computed for the wanted
rows only (:6738-6767); lengths advance after the pass (:6726-6735) and a
step that cannot get its pages changes nothing.

Everything that varies from step to step reaches the kernels through one
block of int32 metadata copied to the device in a single transfer.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Hashable, List, Optional, Sequence

import ctypes
import gc
import itertools

import numpy as np
import torch

from .. import host
from ..cache.pages import CacheManager
from ..cache.storage import CacheStorage
from ..errors import InvalidArgument
from ..parts.base import GroupStep, PhaseTimer, StepContext, StepFacts, StepHost, Workspace


@dataclass
class StepItem:
    """A request's next tokens and the places among them whose logits are wanted."""

    rid: Hashable
    tokens: Sequence[int]
    want: Sequence[int] = field(default_factory=list)
    # the last of `tokens` is not known on the host yet: the device takes the token this request
    # drew in the step before (the value given here is ignored)
    pending_last: bool = False


class _Staging:
    """A few pinned host buffers used in turn, each with the event of its last copy."""

    def __init__(self, device, depth: int = 4):
        self.device = device
        self.depth = depth
        self.host: List[Optional[torch.Tensor]] = [None] * depth
        self.events: List[Optional[torch.cuda.Event]] = [None] * depth
        self.turn = 0

    def next(self, n: int) -> torch.Tensor:
        i = self.turn
        self.turn = (self.turn + 1) % self.depth
        if self.events[i] is not None:
            self.events[i].synchronize()
        buf = self.host[i]
        if buf is None or buf.numel() < n:
            buf = torch.empty(max(n, 1024), dtype=torch.int32, pin_memory=True)
            self.host[i] = buf
        self._last = i
        return buf

    def copied(self) -> None:
        ev = self.events[self._last]
        if ev is None:
            ev = self.events[self._last] = torch.cuda.Event()
        ev.record()


GRAPH_AFTER_MIXED = 3  # eager runs of a shape that its parts do not expect to recur before it is captured


def padded_rows(n: int) -> int:
    """The rows of a step of `n` tokens in which some request brings more than one: the next multiple of
    16 up to 64 rows, of 64 up to 1,024, of 128 beyond. Prompts come in every length, and a step launched
    kernel by kernel costs the host more than the device (GPT-2 small's sizes, a prompt of 512: 0.9 ms of
    launches for 0.75 ms of kernels); in steps of these sizes a prompt's length recurs among a few dozen, so
    that its step is replayed from a captured graph. The products' tiles cover the padding anyway;
    attention and the cache never see it."""
    unit = 16 if n <= 64 else 64 if n <= 1024 else 128
    return -(-n // unit) * unit


class StepFunction:
    """`use_graphs`: a step whose shape (rows, requests, wanted rows, and the key of every
    part's step planner: attention's mode, context bucket and tiles) has been seen before is
    captured into a HIP graph the second time and replayed from then on; what varies between
    such steps lives in the metadata block, whose address and layout the shape fixes. Kernels
    must then depend on the host only through the shape: the ones in this package do. Steps
    that bring prompt portions are padded with rows of no request to sizes that come back
    (`padded_rows`), where every part of the model takes such rows (`pads_rows`)."""

    def __init__(self, model, manager: CacheManager, storage: CacheStorage, device="cuda:0", use_graphs: bool = True,
                 max_graphs: int = 256, batch_invariant: bool = False):
        self.model = model
        self.manager = manager
        self.storage = storage
        self.device = torch.device(device)
        self.workspace = Workspace(self.device)
        self._staging = _Staging(self.device)
        self._meta_dev: Optional[torch.Tensor] = None
        self.steps = 0
        self.tokens = 0
        self.use_graphs = use_graphs
        self.max_graphs = max_graphs
        self.batch_invariant = batch_invariant  # kernels chosen from sizes and positions only (ops.batch_invariant)
        self._graphs = {}  # shape -> (graph, logits) once captured, or the count of eager runs
        self.graph_replays = 0
        self._graph_generation = 0
        self.last_tokens = torch.zeros(manager.max_requests, dtype=torch.int32, device=self.device)
        self.last_context: Optional[StepContext] = None
        self.phases: Optional[PhaseTimer] = None  # set: every step is launched kernel by kernel and timed per phase
        self.planners = list(getattr(model, "step_planners", ()))
        # steps of prompt portions are padded to sizes that recur (padded_rows) where graphs are used and
        # every part of the model takes padding rows
        self.pads_rows = bool(use_graphs and getattr(model, "takes_padding_rows", False))
        self._key = None  # the prepared step's shape: what its captured graph is kept under
        self._recurs = True

    # -- validation -----------------------------------------------------------
    def _validate(self, items: Sequence[StepItem]) -> None:
        if not items:
            raise InvalidArgument("a step needs at least one item")
        seen = set()
        V = self.model.vocab_size
        for it in items:
            if it.rid in seen:
                raise InvalidArgument(f"request {it.rid!r} appears twice in one step")
            seen.add(it.rid)
            if not self.manager.is_open(it.rid):
                raise InvalidArgument(f"request {it.rid!r} is not open")
            n = len(it.tokens)
            if n == 0:
                raise InvalidArgument(f"request {it.rid!r} brings no tokens")
            for w in it.want:
                if not (0 <= int(w) < n):
                    raise InvalidArgument(f"request {it.rid!r} wants logits at place {w} of {n} tokens")
        # a request that would pass the last position is refused by the manager (ContextFull), whose
        # limit is at most the model's learned positions

    # -- eager or replayed ----------------------------------------------------
    def _forward(self, ctx: StepContext) -> Optional[torch.Tensor]:
        from ..kernels import ops

        with ops.batch_invariant(self.batch_invariant):
            return self._run(ctx)

    def _run(self, ctx: StepContext) -> Optional[torch.Tensor]:
        if not self.use_graphs or self.phases is not None:
            ctx.phases = self.phases
            return self.model.forward(ctx, self.storage)
        if self.workspace.generation != self._graph_generation:
            # a workspace buffer moved since the graphs were captured: they hold its old address
            self._graphs.clear()
            self._graph_generation = self.workspace.generation
        key = self._key
        entry = self._graphs.pop(key, None)
        if entry is not None:
            self._graphs[key] = entry  # back in as the most recently used (a dict keeps insertion order)
        if isinstance(entry, tuple):
            entry[0].replay()
            self.graph_replays += 1
            return entry[1]
        if entry is None:
            # first sight: run eagerly, which also sizes every workspace buffer for this shape
            if len(self._graphs) >= self.max_graphs:
                # make room: a shape seen once and never again before a captured graph, the least
                # recently used of either (a serving loop sees many one-off mixes of portions and
                # decoded tokens between its recurring decode-only shapes)
                victim = next((k for k, v in self._graphs.items() if not isinstance(v, tuple)), None)
                self._graphs.pop(victim if victim is not None else next(iter(self._graphs)))
            self._graphs[key] = 1
            return self.model.forward(ctx, self.storage)
        # A decode-only shape comes back step after step: captured at its second sight. A mix of
        # prompt portions and decoded tokens mostly does not, and a capture costs about two eager
        # runs: captured only once it has shown that it recurs.
        if entry < (1 if self._recurs else GRAPH_AFTER_MIXED):
            self._graphs[key] = entry + 1
            return self.model.forward(ctx, self.storage)
        before = self.workspace.generation
        graph = torch.cuda.CUDAGraph()
        # no garbage collection while the stream is capturing: an engine collected then would free
        # pinned memory and events in the middle of the capture, which the runtime answers by aborting
        gc_was_on = gc.isenabled()
        gc.disable()
        try:
            with torch.cuda.graph(graph):
                logits = self.model.forward(ctx, self.storage)
        finally:
            if gc_was_on:
                gc.enable()
        if self.workspace.generation != before:
            # a buffer grew during capture: its old address is baked into the graph; run eagerly
            self._graphs[key] = 1
            return self.model.forward(ctx, self.storage)
        self._graphs[key] = (graph, logits)
        graph.replay()
        self.graph_replays += 1
        return logits

    def forget_graphs(self) -> None:
        """Drops every captured graph and what is known of the shapes seen: the next step of any
        shape is a first sight (measurements of that case use it)."""
        self._graphs.clear()

    # -- the step -------------------------------------------------------------
    def run(self, items: Sequence[StepItem]) -> Optional[torch.Tensor]:
        """Runs the items as one batch from the cache earlier steps left.
        Returns float32 logits [wanted, vocab] on the device, rows in the order
        of the items and of each item's `want`, or None when nothing is wanted.
        The tensor is workspace memory: valid until the next step."""
        ctx, lengths = self.prepare(items, pad=self.pads_rows)
        logits = self._forward(ctx)
        self.commit(items, lengths)
        self.last_context = ctx
        return logits

    def commit(self, items: Sequence[StepItem], lengths) -> None:
        """The requests now hold `lengths` positions (after a step's kernels are enqueued);
        `lengths` is what `prepare` returned for these items."""
        slots, new_lengths = lengths
        self.manager.commit_slots(slots, new_lengths)
        self.steps += 1
        self.tokens += sum(len(it.tokens) for it in items)

    def prepare(self, items: Sequence[StepItem], pad: bool = False):
        """Checks the items, maps their pages (all or nothing) and puts the step's metadata on
        the device. Returns (StepContext, what `commit` needs once the step has run). The
        metadata block is laid out and filled by the host library (csrc/host/step_meta.cpp)
        straight into pinned memory. `pad`: a step in which some request brings more than one token
        gets padding rows behind its tokens up to `padded_rows` of their number (see there)."""
        self._validate(items)
        mgr = self.manager
        S = len(items)
        slots = np.fromiter((mgr.slot(it.rid) for it in items), dtype=np.intc, count=S)
        q_lens = np.fromiter((len(it.tokens) for it in items), dtype=np.intc, count=S)
        want_counts = np.fromiter((len(it.want) for it in items), dtype=np.intc, count=S)
        N, R = int(q_lens.sum()), int(want_counts.sum())
        if all(isinstance(it.tokens, np.ndarray) and it.tokens.ndim == 1 and it.tokens.dtype.kind in "iu" for it in items):
            # arrays of ids (a prompt's portion as the scheduler hands it over) are copied, not walked:
            # 2 us where a list of 2,048 ids takes 70
            all_tokens = np.concatenate([it.tokens for it in items]).astype(np.int64, copy=False)
        else:
            all_tokens = np.fromiter(itertools.chain.from_iterable(it.tokens for it in items), dtype=np.int64, count=N)
        wants = np.fromiter(itertools.chain.from_iterable(it.want for it in items), dtype=np.intc, count=R) if R else \
            np.zeros(1, dtype=np.intc)
        pending = [i for i, it in enumerate(items) if it.pending_last]
        if pending:
            ends = np.cumsum(q_lens) - 1
            all_tokens[ends[pending]] = 0  # checked as a valid id; replaced by a reference below
        if all_tokens.min() < 0 or all_tokens.max() >= self.model.vocab_size:
            bad = int(all_tokens[(all_tokens < 0) | (all_tokens >= self.model.vocab_size)][0])
            raise InvalidArgument(f"token id {bad} is outside [0, {self.model.vocab_size})")  # src/core/transformer.cpp:6195-6197
        if pending:
            all_tokens[ends[pending]] = -1 - slots[pending]  # "the token this slot drew, still on the device"
        new_lengths = mgr.reserve_more(slots, q_lens)

        lib = host.lib()
        shape = host.StepShape()
        ip = lambda a: a.ctypes.data_as(host.IP)  # noqa: E731
        pad_rows = padded_rows(N) - N if pad and N > S and self.phases is None else 0
        host.check(lib.liyab_step_shape(mgr.handle, S, ip(slots), ip(q_lens), ip(want_counts), pad_rows, ctypes.byref(shape)))
        rows = shape.n_rows
        # the parts' own words stand behind the common block; their keys join the step's shape
        first_pos = (new_lengths - q_lens).astype(np.intc, copy=False)
        total = shape.total
        plans = []
        if self.planners:
            facts = StepFacts(n_tokens=N, n_seqs=S, q_lens=q_lens, first_pos=first_pos, state_slots=slots,
                              max_q_len=shape.max_q_len, max_context=shape.max_context, page_size=mgr.page_size)
            for planner in self.planners:
                p = planner.plan(facts)
                plans.append((planner.name, p, total))
                total += p.n_words
        self._key = (rows, S, R) + tuple((name, p.key, p.n_words) for name, p, _ in plans)
        self._recurs = all(p.recurs for _, p, _ in plans)
        host_t = self._staging.next(total)
        base = ctypes.cast(host_t.data_ptr(), ctypes.POINTER(ctypes.c_int32))
        host.check(lib.liyab_step_fill(mgr.handle, ctypes.byref(shape), ip(slots), ip(q_lens),
                                       all_tokens.ctypes.data_as(ctypes.POINTER(ctypes.c_int64)), ip(want_counts), ip(wants),
                                       self.model.vocab_size, base))
        for _, p, off in plans:
            if p.n_words:
                p.fill(ctypes.cast(host_t.data_ptr() + 4 * off, ctypes.POINTER(ctypes.c_int32)))

        if self._meta_dev is None or self._meta_dev.numel() < total:
            # sized for the largest step of this engine's lifetime where possible: a new block
            # would invalidate captured graphs
            self._meta_dev = torch.empty(max(2 * total, 1 << 16), dtype=torch.int32, device=self.device)
            self._graphs.clear()
        dev = self._meta_dev
        dev[:total].copy_(host_t[:total], non_blocking=True)
        self._staging.copied()

        W, G, page = shape.max_blocks, shape.n_groups, mgr.page_size
        starts = np.cumsum(q_lens) - q_lens
        ctx = StepContext(
            n_tokens=rows, n_seqs=S,
            token_ids=dev[shape.off_token_ids:shape.off_token_ids + rows],
            positions=dev[shape.off_positions:shape.off_positions + rows],
            tok_seq=dev[shape.off_tok_seq:shape.off_tok_seq + rows],
            seq_starts=dev[shape.off_seq_starts:shape.off_seq_starts + S + 1],
            context_lens=dev[shape.off_context_lens:shape.off_context_lens + S],
            state_slots=dev[shape.off_state_slots:shape.off_state_slots + S],
            logit_rows=dev[shape.off_logit_rows:shape.off_logit_rows + max(R, 1)], n_logit_rows=R,
            groups=[GroupStep(block_tables=dev[shape.off_block_tables[g]:shape.off_block_tables[g] + S * W].view(S, W),
                              slots=dev[shape.off_slots[g]:shape.off_slots[g] + rows]) for g in range(G)],
            host=StepHost(q_lens=q_lens.tolist(), starts=starts.tolist(), first_pos=first_pos.tolist(),
                          max_q_len=shape.max_q_len, max_context=shape.max_context),
            workspace=self.workspace, dtype=self.model.dtype, page_size=page,
            logit_slots=dev[shape.off_logit_slots:shape.off_logit_slots + max(R, 1)], last_tokens=self.last_tokens,
            plans={name: (p.make(dev[off:off + p.n_words] if p.n_words else None) if p.make is not None else None)
                   for name, p, off in plans},
        )
        return ctx, (slots, new_lengths)
