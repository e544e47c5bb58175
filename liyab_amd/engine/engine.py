"""The engine: requests in, tokens out.

The Python entry point, in the manner of the reference's C++ `Engine`
(include/liyab/engine.h:634-1052): `Engine(model, ...)` for `Engine::create`,
`generate(prompt ids, SamplingParams, on_token)` for `generate_tokens`
(src/core/engine.cpp:3804-3810), statistics named as `GenerationStats`
(include/liyab/types.h:238-292: prompt_tokens, prefill_ms, ttft_ms,
generated_tokens, decode_ms, tokens_per_second, kv_cache_bytes). Where the
reference runs each open sequence on its caller's thread, this engine is
one loop: `add_request` any number of prompts, then `step()` until none is
unfinished; `generate` does that for one or several prompts.
"""

from __future__ import annotations

import time
from dataclasses import dataclass, field
from typing import Callable, Dict, Hashable, List, Optional, Sequence, Union

from ..errors import InvalidArgument
from ..sampling import Sampler, SamplingParams
from .core import EngineCore
from .scheduler import Request, Scheduled, Scheduler
from .step import StepItem


@dataclass
class GenerationStats:
    prompt_tokens: int = 0
    prefill_ms: float = 0.0
    ttft_ms: float = 0.0
    generated_tokens: int = 0
    decode_ms: float = 0.0
    tokens_per_second: float = 0.0
    kv_cache_bytes: int = 0
    preemptions: int = 0


@dataclass
class GenerationResult:
    rid: Hashable
    prompt: List[int]
    tokens: List[int]
    finish_reason: Optional[str]
    stats: GenerationStats = field(default_factory=GenerationStats)


class Engine:
    def __init__(self, model: Optional[str] = None, *, dtype="bfloat16", device="cuda:0", page_size: int = 16,
                 num_pages: Optional[int] = None, max_tokens: Optional[int] = None, max_num_seqs: int = 64,
                 max_batched_tokens: int = 2048, prefill_chunk: int = 256, ctx: Optional[int] = None,
                 overlap: bool = True, use_graphs: bool = True, core: Optional[EngineCore] = None,
                 phases: bool = False, batch_invariant: bool = False):
        """`model`: a folder with config.json and model.safetensors; or `core`: an `EngineCore`
        built elsewhere (`EngineCore.from_plan` for a model made of a plan and tensors), whose
        own dtype, pages and graph setting then hold. `use_graphs`: replay recurring step shapes
        as captured HIP graphs (a part that decides on the host from a step's values, not from
        its shape, needs this off). `batch_invariant`: every reply, greedy or seeded, is the same alone and in any batch in
        bfloat16 too, as the reference promises (include/liyab/engine.h:987-990): kernels are chosen
        from the model's sizes and a token's position only, which costs speed. `phases`: time the device per phase of the forward pass (`phases_ms()`;
        steps are then launched kernel by kernel, so generation is slower). `ctx`: the
        context length (default: the model's). `prefill_chunk`: the longest
        portion of a prompt in one step (the reference's 256,
        src/core/engine.cpp:2863-2864). `num_pages` / `max_tokens` size the
        page pool. `overlap`: schedule and launch the next step before the host has read
        this step's tokens (decoding requests take their last token from a table on the
        device); finishing by an end token is then seen one step late and that step's work
        for the request is dropped. Tokens are the same either way."""
        if core is not None:
            if model is not None:
                raise InvalidArgument("give a model folder or a built core, not both")
            self.core = core
        else:
            self.core = EngineCore(model, dtype=dtype, device=device, page_size=page_size, num_pages=num_pages,
                                   max_tokens=max_tokens, max_requests=max_num_seqs, context_length=ctx,
                                   use_graphs=use_graphs, batch_invariant=batch_invariant)
        self.scheduler = Scheduler(self.core.manager, max_num_seqs=max_num_seqs,
                                   max_batched_tokens=max_batched_tokens, prefill_chunk=prefill_chunk,
                                   eos_token_id=self.core.model.plan.eos_token_id, on_open=self._reset_slot)
        if phases:
            from ..parts.base import PhaseTimer

            self.core.step_fn.phases = PhaseTimer()
        self.sampler = Sampler(self.core.device)
        self._requests: Dict[Hashable, Request] = {}
        self._t_first: Dict[Hashable, float] = {}
        self._t_start: Dict[Hashable, float] = {}
        self._t_end: Dict[Hashable, float] = {}
        self._next_id = 0
        self.stop_at_eos = True
        self.overlap = overlap
        self._inflight = None  # (batch, wanting requests, pinned host tokens, event) of the step not yet read
        self._host_tokens = [None, None]
        self._turn = 0

    def phases_ms(self, reset: bool = False) -> Dict[str, float]:
        """Device milliseconds per phase (embed, attention, dense_ffn, lm_head, ...) summed over the
        steps so far, for an engine made with `phases=True`; the reference's per-phase times
        (include/liyab/types.h:228-236)."""
        timer = self.core.step_fn.phases
        if timer is None:
            return {}
        out = timer.totals()
        if reset:
            timer.reset()
        return out

    def warmup(self) -> None:
        """Runs a short prompt and a few decoded tokens of a request of its own and drops it: the
        first launch of a kernel loads its code, which would otherwise count into the first
        request's time to first token."""
        rid = ("warmup", id(self))
        n = max(1, min(9, self.core.model.max_positions - 4))
        self.core.open(rid)
        try:
            logits = self.core.step([StepItem(rid, [0] * n, [n - 1])])
            for _ in range(3):  # eager, then captured, then replayed
                self.sampler.sample(logits, [SamplingParams(temperature=0.0)], [1], [0])
                self.sampler.sample(logits, [SamplingParams(seed=1)], [1], [0])
                if self.core.manager.length(rid) + 1 >= self.core.model.max_positions:
                    break
                logits = self.core.step([StepItem(rid, [0], [0])])
        finally:
            self.core.close(rid)

    # -- plumbing ---------------------------------------------------------------
    def _reset_slot(self, rid: Hashable) -> None:
        if self.core.storage.states:
            self.core.storage.reset_slot(self.core.manager.slot(rid))

    @property
    def config(self):
        return self.core.config

    # -- continuous batching ------------------------------------------------------
    def add_request(self, prompt_ids: Sequence[int], params: Optional[SamplingParams] = None,
                    rid: Optional[Hashable] = None, priority: int = 0) -> Hashable:
        """`priority`: among waiting requests the larger is admitted first (first come, first
        served among equals); the reference's foreground and background sequences
        (include/liyab/engine.h:1034, 1088-1091) are two values of it."""
        params = params or SamplingParams()
        import numpy as np

        ids = np.asarray(prompt_ids)
        if ids.ndim != 1 or (ids.size and ids.dtype.kind not in "iu"):
            raise InvalidArgument("a prompt is a sequence of token ids")
        V = self.core.vocab_size
        if ids.size and (int(ids.min()) < 0 or int(ids.max()) >= V):
            bad = int(ids[(ids < 0) | (ids >= V)][0])
            raise InvalidArgument(f"token id {bad} is outside [0, {V})")  # src/core/transformer.cpp:6195-6197
        prompt = ids.tolist()
        if rid is None:
            rid = f"req-{self._next_id}"
            self._next_id += 1
        if rid in self._requests and self._requests[rid].state != "finished":
            raise InvalidArgument(f"request {rid!r} is still running")
        r = Request(rid=rid, prompt=prompt, params=params, seed=params.resolved_seed(), priority=int(priority))
        self.scheduler.add(r)
        self._requests[rid] = r
        self._t_first.pop(rid, None)  # an id used before starts its clocks again
        self._t_end.pop(rid, None)
        self._t_start[rid] = time.perf_counter()
        return rid

    def has_unfinished(self) -> bool:
        return self.scheduler.has_unfinished() or self._inflight is not None

    def _resolve(self, inflight, on_token) -> List[Request]:
        """Reads a launched step's tokens and lets the scheduler account for them."""
        batch, wanting, host, event = inflight
        sampled: Dict[Hashable, int] = {}
        if wanting:
            event.synchronize()
            tokens = host[:len(wanting)].tolist()
            now = time.perf_counter()
            for r, t in zip(wanting, tokens):
                sampled[r.rid] = int(t)
                if not r.generated:
                    self._t_first.setdefault(r.rid, now)
        cb = None
        if on_token is not None:
            cb = lambda r, t: on_token(r.rid, t)  # noqa: E731
        saved = self.scheduler.eos_token_id
        if not self.stop_at_eos:
            self.scheduler.eos_token_id = None
        try:
            done = self.scheduler.resolve(batch, sampled, cb)
        finally:
            self.scheduler.eos_token_id = saved
        now = time.perf_counter()
        for r in done:
            self._t_end[r.rid] = now
        return done

    def flush(self, on_token=None) -> List[Request]:
        """Reads the tokens of a step still in flight, if there is one."""
        if self._inflight is None:
            return []
        inflight, self._inflight = self._inflight, None
        return self._resolve(inflight, on_token)

    def step(self, on_token: Optional[Callable[[Hashable, int], Optional[bool]]] = None) -> List[Request]:
        """One scheduler iteration: a batch, a model step, sampling. Returns the requests
        found finished in it (with `overlap`, those of the step before)."""
        import torch

        done: List[Request] = []
        if self._inflight is not None and (not self.overlap or self.scheduler.pressure()):
            done += self.flush(on_token)  # pages are short: no request may carry a pending token into a preemption
        batch = self.scheduler.schedule()
        if not batch:
            return done + self.flush(on_token)
        items = []
        for s in batch:
            r = s.request
            toks = r.token_slice(s.first, s.count)
            items.append(StepItem(r.rid, toks, [s.count - 1] if s.wants_logits else [],
                                  pending_last=r.pending > 0 and s.first + s.count == r.n_tokens))
        logits = self.core.step(items)
        wanting = [s.request for s in batch if s.wants_logits]
        host = event = None
        if wanting:
            ctx = self.core.step_fn.last_context
            host = self._host_tokens[self._turn]
            if host is None or host.numel() < len(wanting):
                host = self._host_tokens[self._turn] = torch.empty(max(64, 2 * len(wanting)), dtype=torch.int32,
                                                                   pin_memory=True)
            self._turn ^= 1
            # the sampling kernel writes the tokens into pinned host memory itself (and into the device's
            # table of last tokens): no copy follows it on the stream
            self.sampler.sample_on_device(
                logits, [r.params for r in wanting], [r.seed for r in wanting],
                [len(r.generated) + r.pending for r in wanting],
                scatter=(ctx.logit_slots, ctx.last_tokens), out=host)
            event = torch.cuda.Event()
            event.record()
        self.scheduler.advance(batch)
        previous, self._inflight = self._inflight, (batch, wanting, host, event)
        if previous is not None:
            done += self._resolve(previous, on_token)
        if not self.overlap:
            done += self.flush(on_token)
        return done

    def abort(self, rid: Hashable) -> None:
        r = self._requests.get(rid)
        if r is not None and r.state != "finished":
            self.scheduler.finish(r, "cancelled")  # a step in flight may still hold it: its result is dropped

    def release(self, rid: Hashable) -> None:
        """Forgets a finished request (its tokens and clocks); `result(rid)` is gone after it."""
        r = self._requests.get(rid)
        if r is not None and r.state == "finished":
            for table in (self._requests, self._t_start, self._t_first, self._t_end):
                table.pop(rid, None)

    def result(self, rid: Hashable) -> GenerationResult:
        r = self._requests[rid]
        end = time.perf_counter()
        t0 = self._t_start.get(rid, end)
        t1 = self._t_first.get(rid, end)
        st = GenerationStats(prompt_tokens=len(r.prompt), generated_tokens=len(r.generated),
                             prefill_ms=(t1 - t0) * 1e3, ttft_ms=(t1 - t0) * 1e3,
                             decode_ms=(self._t_end.get(rid, end) - t1) * 1e3,
                             kv_cache_bytes=self.core.storage.bytes_per_token() * (r.n_tokens - 1),
                             preemptions=r.preemptions)
        if st.decode_ms > 0 and st.generated_tokens > 1:
            # the reference's generated * 1000 / decode_ms (src/core/engine.cpp:4447-4448), over the
            # tokens that decoding steps produced (the first comes out of the prompt's last portion)
            st.tokens_per_second = (st.generated_tokens - 1) * 1000.0 / st.decode_ms
        return GenerationResult(rid=rid, prompt=r.prompt, tokens=list(r.generated), finish_reason=r.finish_reason,
                                stats=st)

    # -- generation ---------------------------------------------------------------
    def generate(self, prompts: Union[Sequence[int], Sequence[Sequence[int]]],
                 params: Union[SamplingParams, Sequence[SamplingParams], None] = None,
                 on_token: Optional[Callable[[Hashable, int], Optional[bool]]] = None):
        """Generates for one prompt (a list of ids -> one GenerationResult) or
        several (a list of lists -> a list of results, batched continuously).
        `on_token(rid, token)` returning False stops that request."""
        single = len(prompts) > 0 and not isinstance(prompts[0], (list, tuple))
        plist = [prompts] if single else list(prompts)
        if not plist:
            raise InvalidArgument("no prompt was given")
        if params is None or isinstance(params, SamplingParams):
            params_list = [params or SamplingParams()] * len(plist)
        else:
            params_list = list(params)
            if len(params_list) != len(plist):
                raise InvalidArgument("one SamplingParams per prompt is needed")
        rids = [self.add_request(p, sp) for p, sp in zip(plist, params_list)]
        while any(self._requests[r].state != "finished" for r in rids):
            self.step(on_token)
        self.flush(on_token)
        results = [self.result(r) for r in rids]
        for r in rids:
            self.release(r)
        return results[0] if single else results
