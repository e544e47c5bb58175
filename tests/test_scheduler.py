"""The scheduler's decisions, with the model replaced by a rule for the next token (no GPU)."""

import pytest

from liyab_amd import InvalidArgument, OutOfPages
from liyab_amd.cache import CacheManager, KVSpec
from liyab_amd.engine.scheduler import FINISHED, RUNNING, WAITING, Request, Scheduler
from liyab_amd.sampling import SamplingParams


def setup(num_pages=64, page_size=16, max_positions=256, max_num_seqs=4, budget=64, chunk=48, eos=None):
    m = CacheManager([(KVSpec(2, 16, 0), [0])], page_size=page_size, num_pages=num_pages, max_requests=8,
                     max_positions=max_positions)
    return m, Scheduler(m, max_num_seqs=max_num_seqs, max_batched_tokens=budget, prefill_chunk=chunk, eos_token_id=eos)


def next_token(r):
    return (sum(r.tokens) * 31 + len(r.tokens)) % 97  # a pure function of the tokens so far


def run(m, s, log=None, limit=10000):
    """Drives the scheduler as the engine does, mapping pages as the step function would."""
    steps = 0
    while s.has_unfinished():
        batch = s.schedule()
        assert batch
        assert sum(b.count for b in batch) <= s.max_batched_tokens
        assert len({b.request.rid for b in batch}) == len(batch)
        m.reserve([(b.request.rid, b.first + b.count) for b in batch])  # never fails: schedule() counted the pages
        for b in batch:
            assert b.first == m.length(b.request.rid) == b.request.computed
            m.commit(b.request.rid, b.first + b.count)
        sampled = {b.request.rid: next_token(b.request) for b in batch if b.wants_logits}
        if log is not None:
            log.append([(b.request.rid, b.first, b.count, b.wants_logits) for b in batch])
        s.update(batch, sampled)
        m.check()
        steps += 1
        assert steps < limit
    return steps


def alone(prompt, max_tokens, max_positions=256):
    r = Request("x", list(prompt), SamplingParams(temperature=0, max_tokens=max_tokens))
    while len(r.generated) < max_tokens and r.n_tokens <= max_positions:
        r.generated.append(next_token(r))
    return r.generated


def test_prompt_portions_decoding_and_finish():
    m, s = setup(budget=64, chunk=48)
    r = Request("a", list(range(100)), SamplingParams(temperature=0, max_tokens=5))
    s.add(r)
    log = []
    run(m, s, log)
    assert [x[0][1:] for x in log[:3]] == [(0, 48, False), (48, 48, False), (96, 4, True)]
    assert all(x[0][2] == 1 and x[0][3] for x in log[3:]) and len(log) == 3 + 4
    assert r.state == FINISHED and r.finish_reason == "length" and r.generated == alone(range(100), 5)
    assert m.pages_in_use() == 0 and not m.is_open("a")
    assert s.stats.batched_tokens == 100 + 4 and s.stats.decode_tokens == 4 and s.stats.prefill_tokens == 100


def test_decodes_first_then_portions_under_the_budget():
    m, s = setup(budget=20, chunk=48)
    a = Request("a", [1, 2, 3], SamplingParams(temperature=0, max_tokens=50))
    s.add(a)
    log = []
    b = Request("b", list(range(60)), SamplingParams(temperature=0, max_tokens=3))
    batch = s.schedule()  # a's prompt alone
    m.reserve([("a", 3)]); m.commit("a", 3); s.update(batch, {"a": next_token(a)})
    s.add(b)
    run(m, s, log)
    first = log[0]
    assert first[0] == ("a", 3, 1, True)  # the decoding request comes first, with its one token
    assert first[1] == ("b", 0, 19, False)  # the portion is what the budget leaves
    assert log[1][1] == ("b", 19, 19, False) and log[3][1] == ("b", 57, 3, True)
    assert a.generated == alone([1, 2, 3], 50) and b.generated == alone(range(60), 3)


def test_admission_first_come_first_served_and_slots():
    m, s = setup(max_num_seqs=2, budget=64, chunk=64)
    rs = [Request(f"r{i}", [i + 1] * 10, SamplingParams(temperature=0, max_tokens=4)) for i in range(4)]
    for r in rs:
        s.add(r)
    batch = s.schedule()
    assert [b.request.rid for b in batch] == ["r0", "r1"] and [r.state for r in rs] == [RUNNING, RUNNING, WAITING, WAITING]
    m.reserve([(b.request.rid, b.count) for b in batch])
    for b in batch:
        m.commit(b.request.rid, b.count)
    s.update(batch, {b.request.rid: next_token(b.request) for b in batch})
    run(m, s)
    assert all(r.generated == alone(r.prompt, 4) for r in rs)


def test_admission_by_priority_then_first_come_first_served():
    """Among waiting requests the higher priority is admitted first, equals in order of arrival
    (the reference lets foreground requests go before background ones, src/core/engine.cpp:1936-1945);
    a preempted request waits ahead of its equals but behind a higher priority."""
    def one_step(m, s):
        batch = s.schedule()
        m.reserve([(b.request.rid, b.first + b.count) for b in batch])
        for b in batch:
            m.commit(b.request.rid, b.first + b.count)
        s.update(batch, {b.request.rid: 9 for b in batch if b.wants_logits})
        m.check()
        return [b.request.rid for b in batch]

    m, s = setup(max_num_seqs=1)
    for rid, pr in (("a", 0), ("b", 0), ("c", 2), ("d", -1), ("e", 2), ("f", 0)):
        s.add(Request(rid, [1, 2, 3], SamplingParams(temperature=0, max_tokens=1), priority=pr))
    assert [r.rid for r in s.waiting] == ["c", "e", "a", "b", "f", "d"]
    order = []
    while s.has_unfinished():
        order += one_step(m, s)
    assert order == ["c", "e", "a", "b", "f", "d"]
    # two requests that cannot both grow to their end in 4 pages: the later one is preempted and
    # waits ahead of its equal, behind the higher priority
    m, s = setup(num_pages=4, max_num_seqs=2)
    first = Request("first", [1] * 30, SamplingParams(temperature=0, max_tokens=30))
    second = Request("second", [1] * 30, SamplingParams(temperature=0, max_tokens=30))
    s.add(first)
    s.add(second)
    one_step(m, s)
    s.add(Request("equal", [1] * 5, SamplingParams(temperature=0, max_tokens=2)))
    s.add(Request("urgent", [1] * 5, SamplingParams(temperature=0, max_tokens=2), priority=1))
    s.add(Request("later", [1] * 5, SamplingParams(temperature=0, max_tokens=2), priority=-3))
    assert [r.rid for r in s.waiting] == ["urgent", "equal", "later"]
    while second.preemptions == 0:
        one_step(m, s)
    # (the step that preempted it admitted the urgent one into the slot it left)
    assert [r.rid for r in s.waiting] == ["second", "equal", "later"] and [r.rid for r in s.running] == ["first", "urgent"]
    while s.has_unfinished():
        one_step(m, s)
    assert len(second.generated) == 30 and len(first.generated) == 30 and m.pages_in_use() == 0


def test_stops_at_eos_and_at_the_last_position():
    m, s = setup(max_positions=32, eos=next_token(Request("p", [5, 6, 7], SamplingParams())))
    r = Request("a", [5, 6, 7], SamplingParams(temperature=0, max_tokens=10))
    s.add(r)
    run(m, s)
    assert r.finish_reason == "stop" and len(r.generated) == 1
    m, s = setup(max_positions=32)
    r = Request("a", list(range(30)), SamplingParams(temperature=0, max_tokens=10))
    s.add(r)
    run(m, s)
    assert r.finish_reason == "context" and len(r.generated) == 3 and r.n_tokens == 33  # positions 0..31 were run
    m, s = setup()
    r = Request("a", [1, 2], SamplingParams(temperature=0, max_tokens=10))
    s.add(r)
    batch = s.schedule()
    m.reserve([("a", 2)]); m.commit("a", 2)
    s.update(batch, {"a": 9}, on_token=lambda req, tok: False)
    assert r.finish_reason == "callback" and m.pages_in_use() == 0


def test_refusals_on_arrival():
    m, s = setup(num_pages=4, max_positions=64)
    with pytest.raises(InvalidArgument, match="empty"):
        s.add(Request("a", [], SamplingParams()))
    with pytest.raises(InvalidArgument, match="max_tokens"):
        s.add(Request("a", [1], SamplingParams(max_tokens=0)))
    with pytest.raises(InvalidArgument, match="context holds"):
        s.add(Request("a", [1] * 65, SamplingParams()))
    m, s = setup(num_pages=2, max_positions=256)
    with pytest.raises(OutOfPages, match="may need 3 pages"):
        s.add(Request("a", [1] * 30, SamplingParams(max_tokens=4)))  # 33 positions > 2 pages: could never fit
    s.add(Request("b", [1] * 30, SamplingParams(max_tokens=3)))  # 32 positions: fits alone


def test_when_pages_run_out_the_latest_request_is_preempted_and_recomputed():
    """8 pages of 16; three requests that each grow to 5 pages cannot all stay. The most recently
    admitted one gives its pages back, waits at the head of the queue and is recomputed from
    its prompt plus what it had generated; everyone's tokens are those it generates alone."""
    m, s = setup(num_pages=8, budget=64, chunk=32, max_num_seqs=3)
    rs = [Request(f"r{i}", [i + 3] * 30, SamplingParams(temperature=0, max_tokens=45)) for i in range(3)]
    for r in rs:
        s.add(r)
    log = []
    run(m, s, log)
    assert s.stats.preemptions >= 1
    assert rs[0].preemptions == 0  # the earliest request is never the victim of a later one
    assert rs[2].preemptions >= 1
    for r in rs:
        assert r.generated == alone(r.prompt, 45), r.rid
        assert r.state == FINISHED
    # a preempted request starts again from position 0 with its generated tokens as prompt
    restarts = [e for step in log for e in step if e[0] == "r2" and e[1] == 0]
    assert len(restarts) == 1 + rs[2].preemptions
    assert s.stats.pages_in_use_peak <= 8 and m.pages_in_use() == 0
    m.check()


def test_no_request_starves_under_pressure():
    m, s = setup(num_pages=6, budget=32, chunk=16, max_num_seqs=4)
    rs = [Request(f"r{i}", [i + 1] * (5 + 7 * i), SamplingParams(temperature=0, max_tokens=30)) for i in range(6)]
    for r in rs:
        s.add(r)
    steps = run(m, s)
    assert steps < 2000
    for r in rs:
        assert r.generated == alone(r.prompt, 30)


def run_lagged(m, s, limit=10000):
    """The engine's overlapped loop: a step's tokens are read only after the next step has been
    scheduled and launched; a request's last token stands as a placeholder meanwhile."""
    inflight, steps = None, 0
    while s.has_unfinished() or inflight is not None:
        if inflight is not None and s.pressure():
            s.resolve(*inflight)
            inflight = None
        batch = s.schedule()
        if not batch:
            assert inflight is not None
            s.resolve(*inflight)
            inflight = None
            continue
        assert sum(b.count for b in batch) <= s.max_batched_tokens
        m.reserve([(b.request.rid, b.first + b.count) for b in batch])
        for b in batch:
            m.commit(b.request.rid, b.first + b.count)
            assert b.request.pending <= 1
        # what the device would sample: a function of the true tokens, which the host learns late
        truth = {}
        for b in batch:
            if b.wants_logits:
                r = b.request
                known = Request("x", r.prompt + r.generated + ([r._late] if r.pending else []), r.params)
                truth[r.rid] = next_token(known)
                r._late = truth[r.rid]
        s.advance(batch)
        previous, inflight = inflight, (batch, truth)
        if previous is not None:
            s.resolve(*previous)
        m.check()
        steps += 1
        assert steps < limit
    return steps


def test_overlapped_loop_gives_the_same_tokens_and_sees_eos_a_step_late():
    prompts = [[3, 4, 5], list(range(40)), [9] * 17, [1]]
    want = [alone(p, 25) for p in prompts]
    eos = want[1][6]  # request 1 stops at its 7th token
    m, s = setup(num_pages=64, budget=32, chunk=16, max_num_seqs=4, eos=eos)
    rs = [Request(f"r{i}", list(p), SamplingParams(temperature=0, max_tokens=25)) for i, p in enumerate(prompts)]
    for r in rs:
        s.add(r)
    run_lagged(m, s)
    for r, w in zip(rs, want):
        cut = w.index(eos) + 1 if eos in w else len(w)
        assert r.generated == w[:cut], r.rid
        assert r.finish_reason == ("stop" if eos in w else "length") and r.pending == 0
    assert m.pages_in_use() == 0 and m.free_slots() == 8
    m.check()


def test_overlapped_loop_under_page_pressure_reads_tokens_before_preempting():
    m, s = setup(num_pages=8, budget=64, chunk=32, max_num_seqs=3)
    rs = [Request(f"r{i}", [i + 3] * 30, SamplingParams(temperature=0, max_tokens=45)) for i in range(3)]
    for r in rs:
        s.add(r)
    run_lagged(m, s)
    assert s.stats.preemptions >= 1
    for r in rs:
        assert r.generated == alone(r.prompt, 45), r.rid
    assert m.pages_in_use() == 0


def test_a_request_at_its_last_token_is_not_scheduled_again():
    m, s = setup(max_positions=32)
    r = Request("a", list(range(30)), SamplingParams(temperature=0, max_tokens=10))
    s.add(r)
    run_lagged(m, s)
    assert r.finish_reason == "context" and len(r.generated) == 3
    m2, s2 = setup()
    r2 = Request("b", [1, 2], SamplingParams(temperature=0, max_tokens=1))
    s2.add(r2)
    batch = s2.schedule()
    m2.reserve([("b", 2)]); m2.commit("b", 2)
    s2.advance(batch)
    assert s2.draining(r2) and s2.schedule() == []  # nothing to run while its only token is pending
    s2.resolve(batch, {"b": 7})
    assert r2.generated == [7] and r2.finish_reason == "length"


def test_token_slice_equals_a_slice_of_tokens():
    import random

    from liyab_amd.engine.scheduler import Request
    from liyab_amd.sampling import SamplingParams

    rng = random.Random(0)
    for _ in range(500):
        r = Request(rid=0, prompt=[rng.randrange(100) for _ in range(rng.randrange(1, 8))], params=SamplingParams())
        r.generated = [rng.randrange(100) for _ in range(rng.randrange(0, 6))]
        r.pending = rng.randrange(0, 3)
        first = rng.randrange(0, r.n_tokens + 1)
        count = rng.randrange(0, r.n_tokens - first + 1)
        assert r.token_slice(first, count) == r.tokens[first:first + count]
        assert len(r.prompt) + len(r.generated) + r.pending == r.n_tokens
    # long portions of a prompt come as arrays of its ids
    for _ in range(100):
        r = Request(rid=0, prompt=[rng.randrange(50000) for _ in range(rng.randrange(64, 400))], params=SamplingParams())
        r.generated = [rng.randrange(100) for _ in range(rng.randrange(0, 6))]
        first = rng.randrange(0, r.n_tokens + 1)
        count = rng.randrange(0, r.n_tokens - first + 1)
        assert list(r.token_slice(first, count)) == r.tokens[first:first + count]


@pytest.mark.parametrize("lagged", [False, True])
@pytest.mark.parametrize("seed", range(6))
def test_native_scheduler_decides_as_the_plain_one(seed, lagged):
    """The same random arrivals, with few pages, through the native scheduler and the plain Python
    one (each on a manager of its own): the same batch at every step, the same queues, the same
    preemptions, the same tokens in the end."""
    import random

    import plain_cache
    import plain_scheduler

    rng = random.Random(500 + seed)
    page_size, num_pages = rng.choice([4, 16]), rng.randint(8, 24)
    kw = dict(page_size=page_size, num_pages=num_pages, max_requests=5, max_positions=120)
    skw = dict(max_num_seqs=rng.randint(2, 5), max_batched_tokens=rng.choice([16, 40, 64]), prefill_chunk=rng.choice([5, 16, 48]))
    arrivals = []
    for i in range(rng.randint(4, 9)):
        n = rng.randint(1, min(60, num_pages * page_size - 1))
        arrivals.append((rng.randint(0, 25), f"q{i}", [rng.randrange(90) for _ in range(n)], rng.randint(1, 40), rng.choice([0, 0, 0, 1, -1, 5])))
    eos = rng.choice([None, 7, 50])

    def drive(native):
        if native:
            m = CacheManager([(KVSpec(2, 16, 0), [0])], **kw)
            s = Scheduler(m, eos_token_id=eos, **skw)
            make = Request
        else:
            m = plain_cache.CacheManager([(plain_cache.KVSpec(2, 16, 0), [0])], **kw)
            s = plain_scheduler.Scheduler(m, eos_token_id=eos, **skw)
            make = plain_scheduler.Request
        log, reqs, pending, inflight, step = [], [], sorted(arrivals), None, 0

        def snapshot(batch):
            log.append(([(b.request.rid, b.first, b.count, b.wants_logits) for b in batch],
                        [r.rid for r in s.running], [r.rid for r in s.waiting], m.free_pages(0),
                        s.stats.preemptions, s.stats.decode_tokens, s.stats.batched_tokens))

        while s.has_unfinished() or inflight is not None or pending:
            while pending and pending[0][0] <= step:
                _, rid, prompt, max_tokens, priority = pending.pop(0)
                r = make(rid, list(prompt), SamplingParams(temperature=0, max_tokens=max_tokens), priority=priority)
                try:
                    s.add(r)
                    reqs.append(r)
                except (InvalidArgument, OutOfPages) as e:
                    log.append(("refused", rid, type(e).__name__))
            step += 1
            if not s.has_unfinished() and inflight is None:
                continue
            if inflight is not None and (not lagged or s.pressure()):
                s.resolve(*inflight)
                inflight = None
                if not s.has_unfinished():
                    continue
            batch = s.schedule()
            snapshot(batch)
            if not batch:
                assert inflight is not None
                s.resolve(*inflight)
                inflight = None
                continue
            m.reserve([(b.request.rid, b.first + b.count) for b in batch])
            truth = {}
            for b in batch:
                m.commit(b.request.rid, b.first + b.count)
                if b.wants_logits:
                    r = b.request
                    known = make("x", r.prompt + r.generated + ([r._late] if r.pending else []), r.params)
                    truth[r.rid] = r._late = next_token(known)
            s.advance(batch)
            previous, inflight = inflight, (batch, truth)
            if previous is not None:
                s.resolve(*previous)
            m.check()
            assert step < 5000
        assert m.pages_in_use(0) == 0
        return log, [(r.rid, r.generated, r.finish_reason, r.preemptions, r.state) for r in reqs]

    native, plain = drive(True), drive(False)
    assert native[0] == plain[0]
    assert native[1] == plain[1]


def test_host_library_under_the_sanitizers(tmp_path):
    """The host C++ (page pools, cache manager, scheduler, a step's metadata) compiled with the
    address and undefined-behaviour sanitizers into a driver of its own that needs no Python,
    and run over random stories of requests: any access out of bounds, use after release or
    overflow ends it with a report."""
    import os
    import subprocess

    from liyab_amd.csrc import build

    exe = build.build_host_selftest(sanitize=True, out_dir=str(tmp_path))
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0", UBSAN_OPTIONS="print_stacktrace=1")
    p = subprocess.run([exe, "120", "120"], capture_output=True, text=True, timeout=300, env=env)
    assert p.returncode == 0, (p.stdout[-2000:], p.stderr[-6000:])
    assert "selftest ok" in p.stdout
