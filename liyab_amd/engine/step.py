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

import itertools

import numpy as np
import torch

from ..cache.pages import UNMAPPED, CacheManager
from ..cache.storage import CacheStorage
from ..errors import ContextFull, InvalidArgument
from ..parts.base import GroupStep, StepContext, StepHost, Workspace


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


ATTN_TILE = 128  # queries of one request that the prefill attention kernel takes together (64 or 128)
DECODE_Q_LEN = 8  # requests that bring at most this many tokens are attended token by token


def _bucket(n: int, least: int = 256) -> int:
    b = least
    while b < n:
        b *= 2
    return b


class StepFunction:
    """`use_graphs`: a step whose shape (tokens, requests, wanted rows, attention mode,
    context bucket) has been seen before is captured into a HIP graph the second time and
    replayed from then on; what varies between such steps lives in the metadata block, whose
    address and layout the shape fixes. Kernels must then depend on the host only through
    the shape: the ones in this package do."""

    def __init__(self, model, manager: CacheManager, storage: CacheStorage, device="cuda:0", use_graphs: bool = True,
                 max_graphs: int = 64):
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
        self._graphs = {}  # shape -> (graph, logits) once captured, or the count of eager runs
        self.graph_replays = 0
        self._graph_generation = 0
        self.last_tokens = torch.zeros(manager.max_requests, dtype=torch.int32, device=self.device)
        self.last_context: Optional[StepContext] = None

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
            end = self.manager.length(it.rid) + n
            if end > self.model.max_positions:
                raise ContextFull(
                    f"position {end - 1} is past the model's {self.model.max_positions} learned positions")

    # -- eager or replayed ----------------------------------------------------
    def _forward(self, ctx: StepContext) -> Optional[torch.Tensor]:
        if not self.use_graphs:
            return self.model.forward(ctx, self.storage)
        if self.workspace.generation != self._graph_generation:
            # a workspace buffer moved since the graphs were captured: they hold its old address
            self._graphs.clear()
            self._graph_generation = self.workspace.generation
        key = (ctx.n_tokens, ctx.n_seqs, ctx.n_logit_rows, ctx.host.attention_mode, ctx.host.context_bucket,
               ctx.host.n_attn_tiles, ctx.host.n_attn_single)
        entry = self._graphs.get(key)
        if isinstance(entry, tuple):
            entry[0].replay()
            self.graph_replays += 1
            return entry[1]
        if entry is None:
            # first sight: run eagerly, which also sizes every workspace buffer for this shape
            if len(self._graphs) >= self.max_graphs:
                self._graphs.pop(next(iter(self._graphs)))
            self._graphs[key] = 1
            return self.model.forward(ctx, self.storage)
        before = self.workspace.generation
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            logits = self.model.forward(ctx, self.storage)
        if self.workspace.generation != before:
            # a buffer grew during capture: its old address is baked into the graph; run eagerly
            self._graphs[key] = 1
            return self.model.forward(ctx, self.storage)
        self._graphs[key] = (graph, logits)
        graph.replay()
        self.graph_replays += 1
        return logits

    # -- the step -------------------------------------------------------------
    def run(self, items: Sequence[StepItem]) -> Optional[torch.Tensor]:
        """Runs the items as one batch from the cache earlier steps left.
        Returns float32 logits [wanted, vocab] on the device, rows in the order
        of the items and of each item's `want`, or None when nothing is wanted.
        The tensor is workspace memory: valid until the next step."""
        ctx, lengths = self.prepare(items)
        logits = self._forward(ctx)
        self.commit(items, lengths)
        self.last_context = ctx
        return logits

    def commit(self, items: Sequence[StepItem], lengths: Sequence[int]) -> None:
        """The requests now hold `lengths` positions (after a step's kernels are enqueued)."""
        for it, n in zip(items, lengths):
            self.manager.commit(it.rid, n)
        self.steps += 1
        self.tokens += sum(len(it.tokens) for it in items)

    def prepare(self, items: Sequence[StepItem]):
        """Checks the items, maps their pages (all or nothing) and puts the step's metadata on
        the device. Returns (StepContext, the lengths to commit once the step has run)."""
        self._validate(items)
        mgr = self.manager
        first = [mgr.length(it.rid) for it in items]
        q_lens = [len(it.tokens) for it in items]
        all_tokens = np.fromiter(itertools.chain.from_iterable(it.tokens for it in items), dtype=np.int64,
                                 count=sum(q_lens))
        if any(it.pending_last for it in items):
            ends = np.cumsum(q_lens) - 1
            for i, it in enumerate(items):
                if it.pending_last:
                    all_tokens[ends[i]] = 0  # checked as a valid id; replaced by a reference below
        if all_tokens.min() < 0 or all_tokens.max() >= self.model.vocab_size:
            bad = int(all_tokens[(all_tokens < 0) | (all_tokens >= self.model.vocab_size)][0])
            raise InvalidArgument(f"token id {bad} is outside [0, {self.model.vocab_size})")  # src/core/transformer.cpp:6195-6197
        for i, it in enumerate(items):
            if it.pending_last:
                all_tokens[ends[i]] = -1 - mgr.slot(it.rid)
        mgr.reserve([(it.rid, f + n) for it, f, n in zip(items, first, q_lens)])

        S, N = len(items), sum(q_lens)
        R = sum(len(it.want) for it in items)
        W = mgr.max_blocks
        G = len(mgr.groups)
        page = mgr.page_size
        starts = np.zeros(S + 1, dtype=np.int64)
        np.cumsum(q_lens, out=starts[1:])

        # attention's work in a step with long portions: tiles of up to 128 queries for them,
        # single rows for requests that bring few tokens
        mode = "decode" if max(q_lens) <= DECODE_Q_LEN else "prefill"
        tiles, singles = [], []
        if mode == "prefill":
            for i, (f, n) in enumerate(zip(first, q_lens)):
                a = int(starts[i])
                if n <= DECODE_Q_LEN:
                    singles.extend(range(a, a + n))
                else:
                    for t0 in range(0, n, ATTN_TILE):
                        tiles.append((i, a + t0, f + t0, min(ATTN_TILE, n - t0)))
            # a tile's work grows with its last position: the longest first, so that the short
            # ones fill the gaps at the end
            tiles.sort(key=lambda t: -(t[2] + t[3]))
            tiles = [v for t in tiles for v in t]
        n_tiles = len(tiles) // 4

        # layout of the metadata block (int32 words)
        off = {}
        cur = 0
        for name, size in (("token_ids", N), ("positions", N), ("tok_seq", N), ("seq_starts", S + 1),
                           ("context_lens", S), ("state_slots", S), ("logit_rows", max(R, 1)),
                           ("logit_slots", max(R, 1)), ("attn_work", max(len(tiles), 1)), ("attn_single", max(len(singles), 1))):
            off[name] = (cur, size)
            cur += size
        for g in range(G):
            off[f"bt{g}"] = (cur, S * W)
            cur += S * W
            off[f"slots{g}"] = (cur, N)
            cur += N
        total = cur
        host_t = self._staging.next(total)
        host = host_t.numpy()

        def view(name):
            o, size = off[name]
            return host[o:o + size]

        tok, pos, seq = view("token_ids"), view("positions"), view("tok_seq")
        rows = view("logit_rows")
        q_arr = np.asarray(q_lens, dtype=np.int64)
        first_arr = np.asarray(first, dtype=np.int64)
        tok[:] = all_tokens
        seq[:] = np.repeat(np.arange(S, dtype=np.int32), q_arr)
        pos[:] = np.repeat(first_arr - starts[:-1], q_arr) + np.arange(N, dtype=np.int64)
        rows[:] = 0
        if R:
            rows[:R] = [int(starts[i]) + int(w) for i, it in enumerate(items) for w in it.want]
        view("seq_starts")[:] = starts
        if tiles:
            view("attn_work")[:] = tiles
        if singles:
            view("attn_single")[:] = singles
        view("context_lens")[:] = first_arr + q_arr
        slot_ids = np.asarray([mgr.slot(it.rid) for it in items], dtype=np.int64)
        view("state_slots")[:] = slot_ids
        if R:
            view("logit_slots")[:R] = [int(slot_ids[i]) for i, it in enumerate(items) for _ in it.want]
        for g in range(G):
            tables = mgr.table_rows(g)[slot_ids]  # [S, W]
            view(f"bt{g}").reshape(S, W)[:] = tables
            pages = tables[seq, pos // page]
            if (pages < 0).any():
                raise AssertionError("a token of this step maps to a released page")
            view(f"slots{g}")[:] = pages * page + pos % page

        if self._meta_dev is None or self._meta_dev.numel() < total:
            # sized for the largest step of this engine's lifetime where possible: a new block
            # would invalidate captured graphs
            self._meta_dev = torch.empty(max(2 * total, 1 << 16), dtype=torch.int32, device=self.device)
            self._graphs.clear()
        dev = self._meta_dev
        dev[:total].copy_(host_t[:total], non_blocking=True)
        self._staging.copied()

        def dview(name):
            o, size = off[name]
            return dev[o:o + size]

        max_context = max(f + n for f, n in zip(first, q_lens))
        ctx = StepContext(
            n_tokens=N, n_seqs=S,
            token_ids=dview("token_ids"), positions=dview("positions"), tok_seq=dview("tok_seq"),
            seq_starts=dview("seq_starts"), context_lens=dview("context_lens"), state_slots=dview("state_slots"),
            logit_rows=dview("logit_rows"), n_logit_rows=R,
            groups=[GroupStep(block_tables=dview(f"bt{g}").view(S, W), slots=dview(f"slots{g}")) for g in range(G)],
            host=StepHost(q_lens=q_lens, starts=[int(s) for s in starts[:-1]], first_pos=first,
                          max_q_len=max(q_lens), max_context=max_context,
                          attention_mode=mode, context_bucket=_bucket(max_context), n_attn_tiles=n_tiles, attn_tile=ATTN_TILE,
                          n_attn_single=len(singles)),
            workspace=self.workspace, dtype=self.model.dtype, page_size=page,
            logit_slots=dview("logit_slots"), last_tokens=self.last_tokens,
            attn_work=dview("attn_work") if mode == "prefill" else None,
            attn_single_rows=dview("attn_single") if mode == "prefill" else None,
        )
        return ctx, [f + n for f, n in zip(first, q_lens)]
