"""The scheduler: admission, prompt portions under a token budget, decoding,
finishing, and what happens when pages run out.

The decisions are native (`csrc/host/scheduler.{h,cpp}`, where the rules and
their sources in the reference are written down: decoding requests first,
then prompt portions under the token budget in order of admission, then
admission by priority, first come first served among equals; when pages run out the most recently
admitted running request is preempted and recomputed later). This module
is their Python face: `Request` objects carry what only the caller knows
(the token ids, the sampling parameters), mirror the counters the native
side keeps for them, and `Scheduler` turns the native batch into
`Scheduled` items for the engine.

The scheduler decides on the host from the cache manager's counts only; it
runs nothing on the GPU and is tested without one.
"""

from __future__ import annotations

import ctypes
from collections import deque
from dataclasses import dataclass, field
from typing import Callable, Deque, Dict, Hashable, List, Optional, Sequence

import numpy as np

from .. import host
from ..cache.pages import CacheManager
from ..errors import InvalidArgument
from ..sampling import SamplingParams

WAITING, RUNNING, FINISHED = "waiting", "running", "finished"
_REASONS = {1: "stop", 2: "length", 3: "context"}


@dataclass
class Request:
    rid: Hashable
    prompt: List[int]
    params: SamplingParams
    seed: int = 0
    generated: List[int] = field(default_factory=list)
    computed: int = 0  # tokens of prompt + generated that are in the cache
    state: str = WAITING
    finish_reason: Optional[str] = None
    preemptions: int = 0
    arrival: int = 0
    pending: int = 0  # tokens sampled in steps whose result the host has not read yet (at most 1 when scheduling)
    sid: int = -1  # the native scheduler's id of this request
    priority: int = 0  # the larger the sooner it is admitted; first come, first served among equals
    _prompt_ids: Optional[np.ndarray] = field(default=None, repr=False, compare=False)  # the prompt as an array, made when a portion is first asked for

    @property
    def tokens(self) -> List[int]:
        """Prompt and generated tokens; a pending token stands as 0 at the end (the device
        knows its value, see StepItem.pending_last)."""
        return self.prompt + self.generated + [0] * self.pending

    def token_slice(self, first: int, count: int):
        """tokens[first:first + count] without putting the whole list together (a decode step
        asks for one token of a long request). A portion of the prompt alone comes as a view of
        an array of its ids, which the step function copies without walking it."""
        n_prompt, end = len(self.prompt), first + count
        if end <= n_prompt:
            if count < 64:
                return self.prompt[first:end]
            if self._prompt_ids is None:
                self._prompt_ids = np.asarray(self.prompt, dtype=np.int64)
            return self._prompt_ids[first:end]
        out = self.prompt[first:] if first < n_prompt else []
        out += self.generated[max(first - n_prompt, 0):end - n_prompt]
        missing = count - len(out)
        return out + [0] * min(missing, self.pending) if missing > 0 else out

    @property
    def n_tokens(self) -> int:
        return len(self.prompt) + len(self.generated) + self.pending

    @property
    def remaining(self) -> int:
        return self.n_tokens - self.computed


@dataclass
class Scheduled:
    request: Request
    first: int  # index of the first token run in this step
    count: int  # how many tokens
    wants_logits: bool  # the portion reaches the request's last token


class Batch(list):
    """A step's `Scheduled` items; `raw` is the native batch they were made from."""

    raw = None
    n_raw = 0


@dataclass
class SchedulerStats:
    steps: int = 0
    batched_tokens: int = 0
    prefill_tokens: int = 0
    decode_tokens: int = 0
    preemptions: int = 0
    pages_in_use_peak: int = 0


class Scheduler:
    def __init__(self, manager: CacheManager, *, max_num_seqs: int, max_batched_tokens: int, prefill_chunk: int,
                 eos_token_id: Optional[int] = None, on_open: Optional[Callable[[Hashable], None]] = None):
        if max_num_seqs <= 0 or max_batched_tokens <= 0 or prefill_chunk <= 0:
            raise InvalidArgument("max_num_seqs, max_batched_tokens and prefill_chunk must be positive")
        self.manager = manager
        self.max_num_seqs = min(max_num_seqs, manager.max_requests)
        self.max_batched_tokens = max_batched_tokens
        self.prefill_chunk = prefill_chunk
        self.eos_token_id = eos_token_id
        self.on_open = on_open
        self._lib = host.lib()
        self._h = self._lib.liyab_sched_create(manager.handle, max_num_seqs, max_batched_tokens, prefill_chunk)
        if not self._h:
            raise InvalidArgument(self._lib.liyab_host_last_error().decode())
        # mirrors of the native queues, as the requests themselves
        self.waiting: Deque[Request] = deque()
        self.running: List[Request] = []
        self._by_sid: Dict[int, Request] = {}
        self._arrivals = 0
        self._peak = 0
        self._raw = ctypes.POINTER(host.Scheduled)()
        self._opened, self._preempted = host.IP(), host.IP()
        self._counts = (ctypes.c_int * 3)()

    def __del__(self):
        if getattr(self, "_h", None):
            self._lib.liyab_sched_destroy(self._h)
            self._h = None

    @property
    def stats(self) -> SchedulerStats:
        out = (ctypes.c_longlong * 5)()
        self._lib.liyab_sched_stats(self._h, out)
        return SchedulerStats(steps=out[0], batched_tokens=out[1], prefill_tokens=out[2], decode_tokens=out[3],
                              preemptions=out[4], pages_in_use_peak=self._peak)

    # -- arrival --------------------------------------------------------------
    def add(self, request: Request) -> None:
        sid = ctypes.c_int(-1)
        try:
            host.check(self._lib.liyab_sched_add(self._h, len(request.prompt), int(request.params.max_tokens),
                                                 int(request.priority), ctypes.byref(sid)))
        except Exception as e:
            raise type(e)(f"request {request.rid!r}: {e}") from None
        request.sid = sid.value
        request.state = WAITING
        request.arrival = self._arrivals
        self._arrivals += 1
        self._by_sid[sid.value] = request
        self._enqueue(request, behind_equals=True)

    def _enqueue(self, request: Request, behind_equals: bool) -> None:
        """Into the waiting queue where the native side puts it: behind every request of a higher
        priority, and behind (a new request) or ahead of (a preempted one) those of its own."""
        at = 0
        for other in self.waiting:
            if other.priority > request.priority or (behind_equals and other.priority == request.priority):
                at += 1
            else:
                break
        self.waiting.insert(at, request)

    def has_unfinished(self) -> bool:
        return bool(self.waiting or self.running)

    def draining(self, r: Request) -> bool:
        """Whether r's pending token is its last whatever it turns out to be: max_tokens
        reached, or no position left to run it at."""
        return r.pending > 0 and (len(r.generated) + r.pending >= r.params.max_tokens or
                                  r.n_tokens > self.manager.max_positions)

    def pressure(self) -> bool:
        """Whether the running requests' next portions may not all fit the free pages, so that
        schedule() may have to preempt; the engine then reads pending tokens first."""
        return bool(self._lib.liyab_sched_pressure(self._h))

    # -- one step's decisions ---------------------------------------------------
    def schedule(self) -> List[Scheduled]:
        """Chooses this step's batch and opens/preempts requests accordingly.
        Pages are only counted here; the step function maps them."""
        rc = self._lib.liyab_sched_schedule(self._h, ctypes.byref(self._raw), ctypes.byref(self._opened),
                                            ctypes.byref(self._preempted), self._counts)
        n, n_opened, n_preempted = self._counts
        # what the native side did to its queues, repeated on the mirrors (preemptions come first)
        for i in range(n_preempted):
            r = self._by_sid[self._preempted[i]]
            self.manager.unbind(r.rid)
            self.running.remove(r)
            r.computed = 0
            r.state = WAITING
            r.preemptions += 1
            self._enqueue(r, behind_equals=False)
        host.check(rc)
        raw = self._raw
        opened = {self._opened[i] for i in range(n_opened)}
        batch = Batch()
        batch.raw, batch.n_raw = raw, n
        by_sid = self._by_sid
        for i in range(n):
            s = raw[i]
            r = by_sid[s.id]
            if s.id in opened:
                self.waiting.popleft()
                r.state = RUNNING
                self.running.append(r)
                self.manager.bind(r.rid, s.slot)
                if self.on_open is not None:
                    self.on_open(r.rid)
            batch.append(Scheduled(r, s.first, s.count, bool(s.wants_logits)))
        return batch

    # -- after the step -----------------------------------------------------------
    def advance(self, batch: Sequence[Scheduled]) -> None:
        """The step has been launched: its tokens are in the cache; requests whose portion
        reached their last token have a token pending."""
        raw, n = getattr(batch, "raw", None), getattr(batch, "n_raw", 0)
        if raw is None or n != len(batch):
            raw = (host.Scheduled * len(batch))(*[host.Scheduled(s.request.sid, self.manager.slot(s.request.rid), s.first,
                                                                 s.count, int(s.wants_logits)) for s in batch])
            n = len(batch)
        self._lib.liyab_sched_advance(self._h, raw, n)
        for s in batch:
            s.request.computed += s.count
            if s.wants_logits:
                s.request.pending += 1

    def resolve(self, batch: Sequence[Scheduled], sampled: Dict[Hashable, int],
                on_token: Optional[Callable[[Request, int], bool]] = None) -> List[Request]:
        """The step's sampled tokens have reached the host; returns requests that finished.
        A request that finished meanwhile (its earlier token ended it while this step was in
        flight) is skipped: what this step computed for it is dropped."""
        wanting = [s.request for s in batch if s.wants_logits]
        done: List[Request] = []
        if wanting:
            tokens = [sampled[r.rid] if r.state != FINISHED else 0 for r in wanting]
            ids = np.fromiter((r.sid for r in wanting), dtype=np.intc, count=len(wanting))
            eos = self.eos_token_id
            stops = np.fromiter((eos is not None and t == eos for t in tokens), dtype=np.intc, count=len(wanting))
            reasons = np.empty(len(wanting), dtype=np.intc)
            ip = lambda a: a.ctypes.data_as(host.IP)  # noqa: E731
            self._lib.liyab_sched_tokens(self._h, ip(ids), ip(stops), len(wanting), ip(reasons))
            for r, token, code in zip(wanting, tokens, reasons.tolist()):
                if code < 0:
                    continue  # finished meanwhile
                r.pending -= 1
                r.generated.append(token)
                reason = _REASONS.get(code)
                if reason is not None:
                    self._finished(r, reason)  # the native side has already let go of it
                if on_token is not None and on_token(r, token) is False and reason is None:
                    reason = "callback"
                    self.finish(r, reason)
                if reason is not None:
                    done.append(r)
        self._peak = max(self._peak, max((g.pool.peak_in_use for g in self.manager.groups), default=0))
        return done

    def update(self, batch: Sequence[Scheduled], sampled: Dict[Hashable, int],
               on_token: Optional[Callable[[Request, int], bool]] = None) -> List[Request]:
        """advance + resolve, for a caller that reads the tokens before the next step."""
        self.advance(batch)
        return self.resolve(batch, sampled, on_token)

    def _finished(self, r: Request, reason: str) -> None:
        if r.state == RUNNING:
            self.manager.unbind(r.rid)
            self.running.remove(r)
        elif r.state == WAITING:
            self.waiting.remove(r)
        r.state = FINISHED
        r.pending = 0
        r.finish_reason = reason
        self._by_sid.pop(r.sid, None)  # the native side has forgotten it too; ids are never given out twice

    def finish(self, r: Request, reason: str) -> None:
        if r.state != FINISHED:
            host.check(self._lib.liyab_sched_finish(self._h, r.sid))
        self._finished(r, reason)
