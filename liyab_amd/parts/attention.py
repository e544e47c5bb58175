"""The attention mixer over paged keys and values."""

from __future__ import annotations

import ctypes
from dataclasses import dataclass
from typing import Optional

import torch

from .. import host
from ..cache.pages import KVSpec
from ..cache.storage import LayerCache
from ..errors import Unsupported
from ..kernels import ops
from .base import PartStepPlan, StepContext, StepFacts, settled
from .linear import linear, linear_deferred, paged_qkv_takes
from .registry import build_part, register_mixer


ATTN_TILE = 128  # queries of one request that the prefill attention kernel takes together (64 or 128)
ATTN_TILE_FEW = 64  # the same for steps whose long portions hold few tokens: more, shorter tiles
ATTN_FEW_TOKENS = 1024  # up to this many tokens in long portions (measured: a step of 256 tokens of one prompt 840 -> 806 us)
DECODE_Q_LEN = 8  # requests that bring at most this many tokens are attended token by token


def attn_tile_for(q_lens) -> int:
    """The query tile of a step's prefill attention. With few tokens in long portions the tiles
    are few, and the longest walk over a request's keys is the whole kernel: tiles of 64
    queries are twice as many, and four waves instead of two share each walk."""
    long_tokens = int(sum(int(q) for q in q_lens if q > DECODE_Q_LEN))
    return ATTN_TILE_FEW if long_tokens <= ATTN_FEW_TOKENS else ATTN_TILE


def _bucket(n: int, least: int = 256) -> int:
    b = least
    while b < n:
        b *= 2
    return b


@dataclass
class AttentionStep:
    """How a step's tokens are attended, decided once a step for every attention layer.
    "decode": every request brings few tokens, each taken on its own. "prefill": the long
    portions in tiles of up to `tile` queries on the matrix cores (`work`: int32 [n_tiles, 4] on
    the device = request index, first row, first position, queries), the short ones' rows
    (`single_rows`: int32 [n_single]) token by token. Grids follow `context_bucket` (the longest
    context rounded up to a power of two), not the exact length."""

    mode: str
    context_bucket: int
    n_tiles: int = 0
    tile: int = ATTN_TILE
    n_single: int = 0
    work: Optional[torch.Tensor] = None
    single_rows: Optional[torch.Tensor] = None


class AttentionStepPlanner:
    """Attention's words of a step's metadata and its term of the graph key: the reference cuts a
    pass's attention into per-segment work the same way, on the host, before its kernels run
    (src/core/transformer.cpp:2169-2174, 2396-2452). The lists are laid out natively
    (csrc/host/attention_plan.cpp: attn_counts, attn_fill)."""

    name = "attention"

    def plan(self, facts: StepFacts) -> PartStepPlan:
        bucket = _bucket(facts.max_context)
        if facts.max_q_len <= DECODE_Q_LEN:
            return PartStepPlan(key=("decode", bucket), make=lambda words: AttentionStep("decode", bucket))
        lib = host.lib()
        tile = attn_tile_for(facts.q_lens)
        counts = (ctypes.c_int * 2)()
        q_lens, first_pos, S = facts.q_lens, facts.first_pos, facts.n_seqs
        lib.liyab_attn_counts(S, q_lens.ctypes.data_as(host.IP), DECODE_Q_LEN, tile, counts)
        n_tiles, n_single = counts[0], counts[1]
        n_work = 4 * max(n_tiles, 1)

        def fill(address) -> None:
            lib.liyab_attn_fill(S, q_lens.ctypes.data_as(host.IP), first_pos.ctypes.data_as(host.IP), DECODE_Q_LEN, tile, address)

        def make(words) -> AttentionStep:
            return AttentionStep("prefill", bucket, n_tiles, tile, n_single, words[:n_work], words[n_work:])

        # a mix of prompt portions mostly does not come back the same
        return PartStepPlan(key=("prefill", bucket, n_tiles, tile, n_single), n_words=n_work + max(n_single, 1), fill=fill,
                            make=make, recurs=False)


class Attention:
    """Causal self-attention with a fused, biased QKV projection and a biased
    output projection: the reference's attention_mixer for a block with
    `fused_qkv` (src/core/transformer.cpp:3083-3140). In order: qkv = h . Wqkv^T
    + b split [q | k | v] (:2657-2673, bias :1263-1273); the step's keys and
    values go to their cache slots before any score is computed, so a portion's
    later tokens see its earlier ones through the cache (:3083-3128); scores,
    softmax and weighted values over positions [0, pos] or the last `window`
    (:2162-2453); out = att . Wo^T + bo added into the residual (:3139-3140,
    :5647). Head counts, head size, scale and window are the spec's; queries
    may outnumber key/value heads by a whole factor. A position encoding of the
    spec's (`spec.position`, a part of the position registry with `rotate(q, k,
    ctx)`) acts on the step's queries and keys in place between the projection
    and the cache write, where the reference applies its rotary encoding
    (:3113-3116); GPT-2 has none."""

    # every launch goes through the kernel library and depends on nothing of this object but its
    # tensors and the constants among its attributes: layers of this kind may run from one recorded list
    replayable = True

    @property
    def takes_padding_rows(self) -> bool:
        """Rows behind the step's tokens (token 0 at position 0 of the first request, slot -1) are computed
        and never read: their keys and values are not written, and no other row attends to them."""
        return self.position is None or bool(getattr(self.position, "takes_padding_rows", False))

    def __init__(self, spec, store, dtype: torch.dtype):
        self.spec = spec
        self.dtype = dtype
        self.width = spec.width
        self.n_head, self.n_kv_head, self.head_dim = spec.n_head, spec.n_kv_head, spec.head_dim
        if self.n_head % self.n_kv_head != 0:
            raise ValueError(f"{self.n_head} query heads are no multiple of {self.n_kv_head} key/value heads")
        if not ops.attention_takes(self.head_dim):
            # said when the model is built, not at its first step
            raise Unsupported(f"attention: heads of {self.head_dim} are not supported (the kernels take head sizes up to "
                              f"{ops.ATTENTION_MAX_HEAD_DIM})")
        self.scale = float(spec.scale)
        self.window = int(spec.window)
        self.q_dim = self.n_head * self.head_dim
        self.kv_dim = self.n_kv_head * self.head_dim
        qkv_out = self.q_dim + 2 * self.kv_dim
        t = spec.tensors
        self.qkv_weight = store.fetch(t["qkv_weight"], (qkv_out, self.width), "matrix")
        self.qkv_bias = store.fetch(t["qkv_bias"], (qkv_out,), "vector") if "qkv_bias" in t else None
        self.out_weight = store.fetch(t["out_weight"], (self.width, self.q_dim), "matrix")
        self.out_bias = store.fetch(t["out_bias"], (self.width,), "vector") if "out_bias" in t else None
        pos = getattr(spec, "position", None)
        self.position = build_part("position", pos, store, dtype) if pos is not None else None
        if self.position is not None and getattr(self.position, "where", None) != "mixer":
            raise ValueError(f"position encoding '{pos.kind}' does not act inside a mixer (where = 'mixer')")

    def cache_spec(self) -> Optional[KVSpec]:
        return KVSpec(self.n_kv_head, self.head_dim, self.window)

    def state_spec(self):
        return None

    defers = True  # forward(..., defer=True) takes the stream split or whole and may hand it back split
    step_planner = AttentionStepPlanner()  # one plan a step for every attention layer: ctx.plans["attention"]

    def forward(self, h: torch.Tensor, ctx: StepContext, cache: LayerCache, state, residual: torch.Tensor,
                writes_cache: bool = True, defer: bool = False):
        """Adds attention's output into `residual`. With `defer`, `residual` may be a SplitStream,
        and where the output projection runs faster cut over its inner dimension the stream
        with the output added comes back as a SplitStream (None: added in place, to the
        stream's own tensor)."""
        n = h.shape[0]
        ws = ctx.workspace
        group = ctx.groups[cache.group]
        if writes_cache and self.position is None and paged_qkv_takes(self.dtype, self.width):
            # the projection's epilogue puts keys and values straight into their pages
            q = ws.get("q", (n, self.q_dim), self.dtype)
            linear(h, self.qkv_weight, self.qkv_bias, out=q, kv=(cache.k, cache.v, group.slots, self.q_dim))
        else:
            q = ws.get("qkv", (n, self.q_dim + 2 * self.kv_dim), self.dtype)
            linear(h, self.qkv_weight, self.qkv_bias, out=q)
            if self.position is not None:
                # queries and keys of this step's tokens, rotated where they lie, before a key is stored
                self.position.rotate(q[:, :self.q_dim], q[:, self.q_dim:self.q_dim + self.kv_dim], ctx)
            if writes_cache:
                ops.kv_write(cache.k, cache.v, q, self.q_dim, self.q_dim + self.kv_dim, group.slots)
        att = ws.get("att", (n, self.q_dim), self.dtype)
        # with few tokens attention may leave each (token, head) pair's keys cut into splits, for
        # an output projection that is cut over its inner dimension and merges them as it loads
        cut = defer and self.dtype == torch.bfloat16 and ops.k_parts(n, self.width, self.q_dim) > 1
        splits = ops.attention(att, q[:, :self.q_dim] if q.shape[1] != self.q_dim else q, cache.k, cache.v, group.block_tables, ctx,
                               n_head=self.n_head, scale=self.scale, window=self.window, splits_ok=cut)
        split = linear_deferred(splits if splits is not None else att, self.out_weight, self.out_bias, ctx, "att_parts", residual) if defer else None
        if split is None:
            if splits is not None:
                ops.attention_merge(att, splits)
            linear(att, self.out_weight, self.out_bias, residual=settled(residual))
        return split


register_mixer("attention", Attention)
