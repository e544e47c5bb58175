"""Schedules for replaying requests through the step function, and the checks
that compare what comes out with the plain implementation."""

from __future__ import annotations

import json
import os
import subprocess
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def stream_tokens(seed, n, vocab):
    """The reference tests' deterministic token stream, tests/test_sequences.cpp:83."""
    return [3 + (t * 37 + seed * 101 + 11) % (vocab - 3) for t in range(n)]


def random_tokens(seed, n, vocab):
    return np.random.default_rng(seed).integers(0, vocab, n).tolist()


# a schedule is a list of steps; a step is {"entries": [(rid, tokens, want)], "end": [rid]}
def schedule_whole(requests):
    return [{"entries": [(rid, toks, list(range(len(toks))))], "end": [rid]} for rid, toks in requests.items()]


def schedule_bulk_tail(requests, tail=32):
    steps = []
    for rid, toks in requests.items():
        bulk = max(0, len(toks) - tail)
        if bulk:
            steps.append({"entries": [(rid, toks[:bulk], list(range(bulk)))], "end": []})
        for i in range(bulk, len(toks)):
            steps.append({"entries": [(rid, toks[i:i + 1], [0])], "end": [rid] if i == len(toks) - 1 else []})
    return steps


def schedule_portions(requests, sizes=(5, 2, 17, 3, 48, 2, 31, 7)):
    steps = []
    for rid, toks in requests.items():
        i, k = 0, 0
        while i < len(toks):
            n = min(sizes[k % len(sizes)], len(toks) - i)
            k += 1
            steps.append({"entries": [(rid, toks[i:i + n], list(range(n)))], "end": [rid] if i + n == len(toks) else []})
            i += n
    return steps


def schedule_mixed(requests, seed=0, max_live=4, decode_tail=12, portions=(2, 9, 5, 17, 3, 48)):
    """Up to `max_live` requests at a time: each runs its tokens in portions of changing size
    until `decode_tail` are left, then one token a step; a new request joins when one ends, so
    portions of some run beside single tokens of others and freed pages are used again."""
    rng = np.random.default_rng(seed)
    pending = list(requests.items())
    live = {}  # rid -> [tokens, done]
    steps = []
    while pending or live:
        while pending and len(live) < max_live:
            rid, toks = pending.pop(0)
            live[rid] = [toks, 0]
            if rng.random() < 0.5:
                break  # join later rather than all at once
        entries, end = [], []
        for rid, (toks, done) in list(live.items()):
            if len(live) > 1 and rng.random() < 0.2:
                continue  # a request may be left out of a step and go on later
            left = len(toks) - done
            n = 1 if left <= decode_tail else min(int(rng.choice(portions)), left - decode_tail)
            n = max(1, n)
            entries.append((rid, toks[done:done + n], list(range(n))))
            live[rid][1] = done + n
            if done + n == len(toks):
                end.append(rid)
        for rid in end:
            del live[rid]
        if entries:
            steps.append({"entries": entries, "end": end})
    return steps


def max_live_tokens(steps, round_to=64):
    """The most tokens live requests hold at any time, each rounded up to `round_to`."""
    held, most = {}, 0
    for st in steps:
        for rid, toks, _ in st["entries"]:
            held[rid] = held.get(rid, 0) + len(toks)
        most = max(most, sum(-(-n // round_to) * round_to for n in held.values()))
        for rid in st["end"]:
            held.pop(rid, None)
    return most


def max_live_pages(steps, page_size):
    """The most pages of `page_size` positions that live requests hold at any time."""
    return max_live_tokens(steps, round_to=page_size) // page_size


def run_schedule(core, steps):
    """Drives an EngineCore through `steps`; returns {rid: {position: float32 logits row}}."""
    from liyab_amd.engine import StepItem

    got, pos = {}, {}
    for st in steps:
        items = []
        for rid, toks, want in st["entries"]:
            if not core.is_open(rid):
                core.open(rid)
                pos[rid] = 0
            items.append(StepItem(rid, toks, want))
        logits = core.step(items)
        if logits is not None:
            rows = logits.float().cpu().numpy()
            r = 0
            for rid, toks, want in st["entries"]:
                for w in want:
                    got.setdefault(rid, {})[pos[rid] + w] = rows[r].copy()
                    r += 1
        for rid, toks, _ in st["entries"]:
            pos[rid] += len(toks)
        for rid in st["end"]:
            core.close(rid)
    return got


def trace_lines(steps):
    out = []
    for i, st in enumerate(steps):
        out.append(json.dumps({"step": i, "entries": [{"id": rid, "tokens": list(map(int, toks)), "want": list(want)}
                                                       for rid, toks, want in st["entries"]], "end": list(st["end"])}))
    return "\n".join(out) + "\n"


def run_trace_program(model_dir, dtype, steps, out_dir, max_tokens, vocab, extra_args=(), env=None):
    """Runs bin/trace_run on `steps`; returns {rid: {position: logits row}} read from its files."""
    cmd = [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", model_dir, "--dtype", dtype, "--out", out_dir,
           "--max-tokens", str(max_tokens), *extra_args]
    p = subprocess.run(cmd, input=trace_lines(steps), capture_output=True, text=True, timeout=600, env=env)
    assert p.returncode == 0, f"trace_run failed ({p.returncode}):\n{p.stdout[-2000:]}\n{p.stderr[-4000:]}"
    done = [l for l in p.stdout.splitlines() if l.startswith("done ")]
    assert done == [f"done {i}" for i in range(len(steps))], p.stdout[-2000:]
    got, pos = {}, {}
    for i, st in enumerate(steps):
        n_want = sum(len(w) for _, _, w in st["entries"])
        path = os.path.join(out_dir, f"{i}.f32")
        if n_want == 0:
            assert not os.path.exists(path)
        else:
            rows = np.fromfile(path, dtype="<f4").reshape(n_want, vocab)
            r = 0
            for rid, toks, want in st["entries"]:
                for w in want:
                    got.setdefault(rid, {})[pos.get(rid, 0) + w] = rows[r]
                    r += 1
        for rid, toks, _ in st["entries"]:
            pos[rid] = pos.get(rid, 0) + len(toks)
    return got


def rel_err(got, ref):
    """max |got - ref| / max |ref| per row; the largest over rows."""
    got = np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    return float((np.abs(got - ref).max(axis=-1) / np.maximum(np.abs(ref).max(axis=-1), 1e-30)).max())


# the largest relative error seen per (family of checks, tolerance): printed at the end of a test
# session (conftest.py), so that the distance between what is observed and what is allowed is on record
WORST = {}


def check_against_plain(got, requests, reference_logits, tol, what="", family=None):
    """Every wanted position of every request within `tol`; names the first wrong one."""
    worst = 0.0
    key = (family or what.split(" ")[0] or "logits", tol)
    for rid, toks in requests.items():
        ref = reference_logits[rid]
        assert rid in got, f"{what}: no logits for request {rid}"
        for p in sorted(got[rid]):
            row = got[rid][p]
            assert np.isfinite(row).all(), f"{what}: request {rid} position {p}: non-finite logits"
            e = rel_err(row, ref[p])
            worst = max(worst, e)
            WORST[key] = max(WORST.get(key, 0.0), e)
            assert e <= tol, (f"{what}: request {rid} (length {len(toks)}) first differs at position {p}: "
                              f"relative error {e:.3e} > {tol:.1e}")
    return worst
