"""A plain scheduler in Python: the reference the native one (liyab_amd/csrc/host/scheduler.cpp)
is compared with, decision by decision, in tests/test_scheduler.py. The rules are those written
at the top of csrc/host/scheduler.h (decoding requests first, prompt portions under the token
budget in order of admission, first come first served admission, preemption of the most recently
admitted request when pages run out); the reference's own scheduling is by threads
(src/core/engine.cpp:1842-2041) with portions of 256 tokens (:2863-2864) and the stop rules of
:4351-4393. It shares no code with the product (it runs on a manager of its own)."""

from __future__ import annotations

from collections import deque
from dataclasses import dataclass, field
from typing import Callable, Deque, Dict, Hashable, List, Optional, Sequence

from liyab_amd.errors import InvalidArgument, OutOfPages
from liyab_amd.sampling import SamplingParams

WAITING, RUNNING, FINISHED = "waiting", "running", "finished"


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
    priority: int = 0  # the larger the sooner it is admitted

    @property
    def tokens(self) -> List[int]:
        """Prompt and generated tokens; a pending token stands as 0 at the end (the device
        knows its value, see StepItem.pending_last)."""
        return self.prompt + self.generated + [0] * self.pending

    def token_slice(self, first: int, count: int) -> List[int]:
        """tokens[first:first + count] without putting the whole list together (a decode step
        asks for one token of a long request)."""
        n_prompt, end = len(self.prompt), first + count
        if end <= n_prompt:
            return self.prompt[first:end]
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


@dataclass
class SchedulerStats:
    steps: int = 0
    batched_tokens: int = 0
    prefill_tokens: int = 0
    decode_tokens: int = 0
    preemptions: int = 0
    pages_in_use_peak: int = 0


class Scheduler:
    def __init__(self, manager, *, max_num_seqs: int, max_batched_tokens: int, prefill_chunk: int,
                 eos_token_id: Optional[int] = None, on_open: Optional[Callable[[Hashable], None]] = None):
        if max_num_seqs <= 0 or max_batched_tokens <= 0 or prefill_chunk <= 0:
            raise InvalidArgument("max_num_seqs, max_batched_tokens and prefill_chunk must be positive")
        self.manager = manager
        self.max_num_seqs = min(max_num_seqs, manager.max_requests)
        self.max_batched_tokens = max_batched_tokens
        self.prefill_chunk = prefill_chunk
        self.eos_token_id = eos_token_id
        self.on_open = on_open
        self.waiting: Deque[Request] = deque()
        self.running: List[Request] = []
        self.stats = SchedulerStats()
        self._arrivals = 0

    # -- arrival --------------------------------------------------------------
    def add(self, request: Request) -> None:
        if not request.prompt:
            raise InvalidArgument("the prompt is empty")  # src/core/engine.cpp:3867-3871
        if request.params.max_tokens <= 0:
            raise InvalidArgument("max_tokens must be positive")
        if len(request.prompt) >= self.manager.max_positions + 1:
            raise InvalidArgument(
                f"the prompt has {len(request.prompt)} tokens; the context holds {self.manager.max_positions}")
        # the most positions it can come to hold: every token but the last sampled one is run
        most = min(len(request.prompt) + request.params.max_tokens - 1, self.manager.max_positions)
        need = -(-most // self.manager.page_size)
        for g in self.manager.groups:
            if g.spec.window <= 0 and need > g.pool.num_pages:
                raise OutOfPages(
                    f"request {request.rid!r} may need {need} pages; the pool has {g.pool.num_pages} in all")
        request.state = WAITING
        request.arrival = self._arrivals
        self._arrivals += 1
        self._enqueue(request, behind_equals=True)

    def _enqueue(self, request, behind_equals: bool) -> None:
        """Behind every waiting request of a higher priority, and behind (a new request) or ahead
        of (a preempted one) those of its own: foreground before background as the reference
        chooses a pass's requests (src/core/engine.cpp:1936-1945), first come first served among equals."""
        queue = list(self.waiting)
        keep = [o for o in queue if o.priority > request.priority or (behind_equals and o.priority == request.priority)]
        assert queue[:len(keep)] == keep  # the queue is ordered by priority
        self.waiting.insert(len(keep), request)

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
        groups = self.manager.groups
        free = min(g.pool.free_pages for g in groups)
        page, chunk = self.manager.page_size, self.prefill_chunk
        # a portion of c tokens takes at most ceil(c / page) + 1 new pages of a group
        bound = 0
        for r in self.running:
            count = min(r.remaining, chunk)
            if count > 0:
                bound += -(-count // page) + 1
        if bound <= free:
            return False
        need = [0] * len(groups)
        for r in self.running:
            count = min(r.remaining, chunk)
            if count <= 0:
                continue
            for gi, n in enumerate(self.manager.pages_needed(r.rid, r.computed + count)):
                need[gi] += n
        return any(n > g.pool.free_pages for n, g in zip(need, groups))

    # -- one step's decisions ---------------------------------------------------
    def _open(self, r: Request) -> None:
        self.manager.open(r.rid)
        if self.on_open is not None:
            self.on_open(r.rid)

    def _preempt(self, r: Request) -> None:
        if r.pending > 0:
            raise AssertionError("a request with a pending token cannot be preempted: read the tokens first")
        self.manager.close(r.rid)
        self.running.remove(r)
        r.computed = 0
        r.state = WAITING
        r.preemptions += 1
        self.stats.preemptions += 1
        self._enqueue(r, behind_equals=False)

    def schedule(self) -> List[Scheduled]:
        """Chooses this step's batch and opens/preempts requests accordingly.
        Pages are only counted here; the step function maps them."""
        budget = self.max_batched_tokens
        batch: List[Scheduled] = []
        groups = self.manager.groups
        need = [0] * len(groups)  # pages this step's batch takes so far, per group

        page, n_groups = self.manager.page_size, len(groups)

        def extra(r: Request, count: int) -> List[int]:
            # new pages per group for positions [computed, computed + count): the request's pages
            # reach its computed length at least, so this never undercounts
            return [-(-(r.computed + count) // page) - (-(-r.computed // page))] * n_groups

        free = [g.pool.free_pages for g in groups]  # read again whenever a request is opened or preempted

        def fits(r: Request, count: int, pages: Optional[List[int]] = None) -> bool:
            return all(n + e <= f for n, e, f in zip(need, pages or extra(r, count), free))

        def take(r: Request, count: int, pages: Optional[List[int]] = None) -> None:
            nonlocal budget
            for gi, e in enumerate(pages or extra(r, count)):
                need[gi] += e
            batch.append(Scheduled(r, r.computed, count, r.computed + count == r.n_tokens))
            budget -= count

        def untake(s: Scheduled) -> None:
            nonlocal budget
            for gi, e in enumerate(extra(s.request, s.count)):
                need[gi] -= e
            batch.remove(s)
            budget += s.count

        # running requests: decoding ones first, then prompt portions, each in order of admission
        active = [r for r in self.running if not self.draining(r)]
        order = [r for r in active if r.remaining == 1] + [r for r in active if r.remaining > 1]
        for r in order:
            if r.state != RUNNING or budget <= 0:
                continue
            count = min(r.remaining, self.prefill_chunk, budget)
            pages = extra(r, count)  # counted once on the common path, where everything fits
            if fits(r, count, pages):
                take(r, count, pages)
                continue
            while not fits(r, count):
                victim = self.running[-1]
                if victim is r:
                    # nobody later to take pages from: shrink the portion or wait
                    while count > 1 and not fits(r, count):
                        count -= 1
                    if not fits(r, count):
                        count = 0
                    break
                for s in [s for s in batch if s.request is victim]:
                    untake(s)
                self._preempt(victim)
                free[:] = [g.pool.free_pages for g in groups]
            if count > 0 and r.state == RUNNING:
                take(r, count)
        # admission, first come first served
        while self.waiting and len(self.running) < self.max_num_seqs and budget > 0:
            r = self.waiting[0]
            count = min(r.remaining, self.prefill_chunk, budget)
            pages = -(-count // self.manager.page_size)
            if self.manager.free_slots() == 0 or any(n + pages > f for n, f in zip(need, free)):
                break
            self._open(r)
            self.waiting.popleft()
            r.state = RUNNING
            self.running.append(r)
            take(r, count)
        if not batch and self.has_unfinished() and not any(r.pending > 0 for r in self.running):
            raise OutOfPages("no request can make progress: the page pool is too small for any of them")
        self.stats.steps += 1
        n = sum(s.count for s in batch)
        self.stats.batched_tokens += n
        self.stats.decode_tokens += sum(1 for s in batch if s.count == 1 and s.wants_logits and s.request.generated)
        self.stats.prefill_tokens = self.stats.batched_tokens - self.stats.decode_tokens
        return batch

    # -- after the step -----------------------------------------------------------
    def advance(self, batch: Sequence[Scheduled]) -> None:
        """The step has been launched: its tokens are in the cache; requests whose portion
        reached their last token have a token pending."""
        for s in batch:
            s.request.computed += s.count
            if s.wants_logits:
                s.request.pending += 1

    def resolve(self, batch: Sequence[Scheduled], sampled: Dict[Hashable, int],
                on_token: Optional[Callable[[Request, int], bool]] = None) -> List[Request]:
        """The step's sampled tokens have reached the host; returns requests that finished.
        A request that finished meanwhile (its earlier token ended it while this step was in
        flight) is skipped: what this step computed for it is dropped."""
        done = []
        for s in batch:
            r = s.request
            if not s.wants_logits or r.state == FINISHED:
                continue
            token = sampled[r.rid]
            r.pending -= 1
            r.generated.append(token)
            reason = None
            if self.eos_token_id is not None and token == self.eos_token_id:
                reason = "stop"
            elif len(r.generated) >= r.params.max_tokens:
                reason = "length"
            elif len(r.prompt) + len(r.generated) > self.manager.max_positions:
                reason = "context"  # the next token would pass the last position
            if on_token is not None and on_token(r, token) is False and reason is None:
                reason = "callback"
            if reason is not None:
                self.finish(r, reason)
                done.append(r)
        self.stats.pages_in_use_peak = max(self.stats.pages_in_use_peak,
                                           max((g.pool.peak_in_use for g in self.manager.groups), default=0))
        return done

    def update(self, batch: Sequence[Scheduled], sampled: Dict[Hashable, int],
               on_token: Optional[Callable[[Request, int], bool]] = None) -> List[Request]:
        """advance + resolve, for a caller that reads the tokens before the next step."""
        self.advance(batch)
        return self.resolve(batch, sampled, on_token)

    def finish(self, r: Request, reason: str) -> None:
        if r.state == RUNNING:
            self.manager.close(r.rid)
            self.running.remove(r)
        elif r.state == WAITING:
            self.waiting.remove(r)
        r.state = FINISHED
        r.pending = 0
        r.finish_reason = reason
