"""The engine against the plain implementation, under every way of cutting and batching the
work, in 32-bit and in bfloat16 (needs the GPU)."""

import json
import os
import subprocess
import sys

import numpy as np
import pytest

import plain_gpt2 as plain
import trace_tools as tt
from conftest import CONFIGS, ROOT, TOL

pytestmark = pytest.mark.gpu

DTYPES = ["float32", "bfloat16"]


def make_requests(name):
    """Token sequences of the workloads: prompt + continuation, teacher-forced."""
    cfg, _ = CONFIGS[name]
    V, P = cfg["vocab_size"], cfg["n_positions"]
    if name == "A":
        lens = {"a0": 7 + 24, "a1": 19 + 24, "a2": 1 + 24, "a3": P, "a4": 70}
        seed = 1
    else:
        lens = {"b0": 1 + 32, "b1": 13 + 32, "b2": 64 + 32, "b3": 100 + 32, "b4": 200 + 32, "b5": P}
        seed = 3
    reqs = {}
    for i, (rid, n) in enumerate(lens.items()):
        reqs[rid] = tt.random_tokens(seed * 100 + i, n, V) if i != 4 else tt.stream_tokens(seed, n, V)
    return reqs


@pytest.fixture(scope="module")
def reference(plain_models):
    """{(model, dtype): {rid: logits [T, V]}} from the plain implementation. The bfloat16 path
    holds its matrices in bfloat16, so its reference uses the matrices rounded the same way."""
    out = {}
    for name in ("A", "B"):
        config, tensors = plain_models[name]
        reqs = make_requests(name)
        out[(name, "float32")] = {rid: plain.forward(config, tensors, toks) for rid, toks in reqs.items()}
        rounded = plain.round_weights_to_bf16(tensors)
        out[(name, "bfloat16")] = {rid: plain.forward(config, rounded, toks) for rid, toks in reqs.items()}
    return out


def make_core(model_dir, dtype, max_tokens, page_size=16, poison=True, num_pages=None):
    import torch

    from liyab_amd.engine import EngineCore

    core = EngineCore(model_dir, dtype=dtype, page_size=page_size, max_tokens=max_tokens, num_pages=num_pages, max_requests=8)
    if poison:  # free pages hold NaN: a kernel that reads past a request's length shows it
        for c in core.storage.layers.values():
            for t in c.rows.values():
                t.fill_(float("nan"))
        torch.cuda.synchronize()
    return core


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B"])
def test_each_request_alone_and_whole(name, dtype, model_dirs, reference):
    reqs = make_requests(name)
    steps = tt.schedule_whole(reqs)
    core = make_core(model_dirs[name], dtype, tt.max_live_tokens(steps))
    got = tt.run_schedule(core, steps)
    for rid, toks in reqs.items():
        assert sorted(got[rid]) == list(range(len(toks)))
    tt.check_against_plain(got, reqs, reference[(name, dtype)], TOL[dtype], f"whole {name} {dtype}")
    core.manager.check()
    assert core.manager.pages_in_use() == 0


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B"])
def test_bulk_then_last_32_one_by_one(name, dtype, model_dirs, reference):
    reqs = make_requests(name)
    steps = tt.schedule_bulk_tail(reqs, tail=32)
    core = make_core(model_dirs[name], dtype, tt.max_live_tokens(steps))
    got = tt.run_schedule(core, steps)
    tt.check_against_plain(got, reqs, reference[(name, dtype)], TOL[dtype], f"bulk+tail {name} {dtype}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B"])
@pytest.mark.parametrize("sizes", [(5,), (48,), (5, 2, 17, 3, 48, 2, 31, 7)])
def test_portions_of_changing_size(name, dtype, sizes, model_dirs, reference):
    reqs = make_requests(name)
    steps = tt.schedule_portions(reqs, sizes)
    core = make_core(model_dirs[name], dtype, tt.max_live_tokens(steps))
    got = tt.run_schedule(core, steps)
    tt.check_against_plain(got, reqs, reference[(name, dtype)], TOL[dtype], f"portions {sizes} {name} {dtype}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B"])
@pytest.mark.parametrize("seed", [0, 1])
def test_mixed_batches_with_pages_used_again(name, dtype, seed, model_dirs, reference):
    reqs = make_requests(name)
    steps = tt.schedule_mixed(reqs, seed=seed)
    assert any(len(st["entries"]) >= 2 for st in steps), "no step held several requests"
    assert any(len(st["entries"]) >= 2 and {len(t) for _, t, _ in st["entries"]} > {1} and
               any(len(t) == 1 for _, t, _ in st["entries"]) for st in steps), "no step mixed a portion with a single token"
    most = tt.max_live_tokens(steps)
    total = sum(-(-len(t) // 64) * 64 for t in reqs.values())
    assert most < total, "the pool would hold every request at once: no page would be used again"
    core = make_core(model_dirs[name], dtype, most)
    got = tt.run_schedule(core, steps)
    tt.check_against_plain(got, reqs, reference[(name, dtype)], TOL[dtype], f"mixed {name} {dtype}")
    core.manager.check()
    assert core.manager.pages_in_use() == 0


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name,page_size", [("A", 24), ("B", 48), ("B", 3)])
def test_mixed_batches_with_pages_that_are_no_power_of_two(name, page_size, dtype, model_dirs, reference):
    """Pages of 24, 48 and 3 positions (the reference takes any page_tokens,
    include/liyab/kv_cache.h:72-80): page and offset by division in every kernel that looks a
    position up, with just the pages the schedule needs, so that they are used again."""
    reqs = make_requests(name)
    steps = tt.schedule_mixed(reqs, seed=3)
    pages = tt.max_live_pages(steps, page_size)
    assert pages < sum(-(-len(t) // page_size) for t in reqs.values())
    core = make_core(model_dirs[name], dtype, None, page_size=page_size, num_pages=pages)
    got = tt.run_schedule(core, steps)
    tt.check_against_plain(got, reqs, reference[(name, dtype)], TOL[dtype], f"mixed, pages of {page_size}, {name} {dtype}", family="mixed")
    core.manager.check()
    assert core.manager.pages_in_use() == 0
    # whole prompts through the tiled attention kernel, too
    steps = tt.schedule_whole(reqs)
    core = make_core(model_dirs[name], dtype, None, page_size=page_size, num_pages=tt.max_live_pages(steps, page_size))
    got = tt.run_schedule(core, steps)
    tt.check_against_plain(got, reqs, reference[(name, dtype)], TOL[dtype], f"whole, pages of {page_size}, {name} {dtype}", family="whole")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B"])
def test_long_decoding_from_the_first_token(name, dtype, model_dirs, reference):
    """Every token of the longest request one by one, from position 0 to the last position."""
    reqs = make_requests(name)
    rid = "a3" if name == "A" else "b5"
    one = {rid: reqs[rid]}
    steps = tt.schedule_bulk_tail(one, tail=len(one[rid]))
    core = make_core(model_dirs[name], dtype, tt.max_live_tokens(steps))
    got = tt.run_schedule(core, steps)
    tt.check_against_plain(got, one, reference[(name, dtype)], TOL[dtype], f"decode all {name} {dtype}")
    # the first tokens of a sequence: position 0 attends to itself only
    assert sorted(got[rid])[:4] == [0, 1, 2, 3]


@pytest.mark.parametrize("dtype", DTYPES)
def test_context_full_and_bad_ids(dtype, model_dirs):
    from liyab_amd import ContextFull, InvalidArgument
    from liyab_amd.engine import StepItem

    cfg, _ = CONFIGS["A"]
    core = make_core(model_dirs["A"], dtype, 256)
    core.open("x")
    core.step([StepItem("x", [1] * cfg["n_positions"], [])])
    with pytest.raises(ContextFull):
        core.step([StepItem("x", [1], [0])])
    core.open("y")
    with pytest.raises(InvalidArgument):
        core.step([StepItem("y", [cfg["vocab_size"]], [0])])
    with pytest.raises(InvalidArgument):
        core.step([StepItem("y", [], [])])
    with pytest.raises(InvalidArgument):
        core.step([StepItem("y", [1], [0]), StepItem("y", [2], [0])])
    assert core.length("y") == 0


def test_out_of_pages_changes_nothing(model_dirs):
    from liyab_amd import OutOfPages
    from liyab_amd.engine import StepItem

    core = make_core(model_dirs["A"], "float32", 64)  # 4 pages of 16
    core.open("x")
    core.open("y")
    core.step([StepItem("x", [1] * 40, [])])
    before = core.manager.pages_in_use()
    with pytest.raises(OutOfPages):
        core.step([StepItem("x", [2], [0]), StepItem("y", [3] * 20, [])])
    assert core.manager.pages_in_use() == before and core.length("x") == 40 and core.length("y") == 0
    core.manager.check()


def test_truncate_and_replay_gives_the_same_logits(model_dirs, plain_models):
    """The reference's rollback check: 70 tokens, back to 65, the last 5 again
    (tests/test_engine.cpp:3740-3741, 3764-3767)."""
    cfg, _ = CONFIGS["B"]
    toks = [3 + (i * 37) % 280 for i in range(70)]
    core = make_core(model_dirs["B"], "float32", 128)
    from liyab_amd.engine import StepItem

    core.open("r")
    first = core.step([StepItem("r", toks, list(range(70)))]).cpu().numpy().copy()
    core.truncate("r", 65)
    again = core.step([StepItem("r", toks[65:], list(range(5)))]).cpu().numpy()
    assert tt.rel_err(again, first[65:]) <= TOL["float32"]
    config, tensors = plain_models["B"]
    assert tt.rel_err(first, plain.forward(config, tensors, toks)) <= TOL["float32"]


@pytest.mark.parametrize("dtype", DTYPES)
def test_trace_program_mixed(dtype, model_dirs, reference, tmp_path):
    """bin/trace_run as a user runs it: a mixed trace with few pages, its files compared."""
    name = "B"
    cfg, _ = CONFIGS[name]
    reqs = make_requests(name)
    steps = tt.schedule_mixed(reqs, seed=2)
    # some steps want nothing, some want a few places
    for st in steps[::3]:
        st["entries"] = [(rid, toks, want[-1:]) for rid, toks, want in st["entries"]]
    steps[1]["entries"] = [(rid, toks, []) for rid, toks, want in steps[1]["entries"]]
    got = tt.run_trace_program(model_dirs[name], dtype, steps, str(tmp_path / "out"), tt.max_live_tokens(steps),
                               cfg["vocab_size"])
    tt.check_against_plain(got, reqs, reference[(name, dtype)], TOL[dtype], f"trace_run {dtype}")


def _near_argmax(ref_row, token, tol):
    ref_row = np.asarray(ref_row, dtype=np.float64)
    return ref_row[token] >= ref_row.max() - tol * np.abs(ref_row).max()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B"])
def test_greedy_generation_through_the_entry_point(name, dtype, model_dirs, plain_models):
    """Engine.generate with several prompts batched continuously; each token is the plain
    implementation's greedy choice given the tokens so far (or within tolerance of it)."""
    from liyab_amd import Engine, SamplingParams

    cfg, _ = CONFIGS[name]
    config, tensors = plain_models[name]
    if dtype == "bfloat16":
        tensors = plain.round_weights_to_bf16(tensors)
    V = cfg["vocab_size"]
    n_new = 24 if name == "A" else 32
    lens = [7, 19, 1] if name == "A" else [1, 13, 64, 100, 200]
    prompts = [tt.random_tokens(40 + i, n, V) for i, n in enumerate(lens)]
    engine = Engine(model_dirs[name], dtype=dtype, page_size=16, num_pages=40, max_num_seqs=4, max_batched_tokens=64,
                    prefill_chunk=5 if name == "A" else 48)
    engine.stop_at_eos = False
    if name == "B":  # a warm-up beforehand leaves nothing behind
        engine.warmup()
        assert engine.core.manager.pages_in_use() == 0
    results = engine.generate(prompts, SamplingParams(temperature=0.0, max_tokens=n_new))
    for prompt, res in zip(prompts, results):
        want_n = min(n_new, cfg["n_positions"] - len(prompt) + 1)
        assert len(res.tokens) == want_n and res.finish_reason in ("length", "context")
        ref = plain.forward(config, tensors, prompt + res.tokens[:-1])
        for i, t in enumerate(res.tokens):
            row = ref[len(prompt) - 1 + i]
            assert _near_argmax(row, t, TOL[dtype]), f"token {i} of prompt length {len(prompt)}: {t} vs {int(np.argmax(row))}"
        if dtype == "float32":
            assert res.tokens == plain.generate_greedy(config, tensors, prompt, n_new)
    assert engine.core.manager.pages_in_use() == 0
    engine.core.manager.check()


@pytest.mark.parametrize("dtype", DTYPES)
def test_temperature_sampling_alone_and_batched(dtype, model_dirs, plain_models):
    """Temperature 0.8, sampler seed 4: the same tokens alone and in a batch, and each the
    plain sampler's draw from the plain logits (unless the draw falls on a boundary)."""
    from liyab_amd import Engine, SamplingParams

    name = "B"
    cfg, _ = CONFIGS[name]
    config, tensors = plain_models[name]
    V = cfg["vocab_size"]
    prompts = [tt.random_tokens(60 + i, n, V) for i, n in enumerate([1, 13, 64])]
    sp = SamplingParams(temperature=0.8, top_k=0, top_p=1.0, seed=4, max_tokens=32)
    engine = Engine(model_dirs[name], dtype=dtype, page_size=16, max_num_seqs=4, max_batched_tokens=64, prefill_chunk=48)
    engine.stop_at_eos = False
    together = engine.generate(prompts, sp)
    alone = [engine.generate(p, sp) for p in prompts]
    for a, b in zip(together, alone):
        assert a.tokens == b.tokens
    if dtype == "float32":
        for prompt, res in zip(prompts, together):
            ref = plain.forward(config, tensors, prompt + res.tokens[:-1])
            for i, t in enumerate(res.tokens):
                probs = plain.probabilities(ref[len(prompt) - 1 + i], 0.8)
                u = plain.uniform(4, i)
                expect = plain.sample(probs, u)
                if t != expect:
                    cdf = np.cumsum(probs)
                    assert np.abs(cdf - u).min() < 1e-5, f"token {i}: {t} vs {expect}, not a boundary case"


def test_command_line_json(model_dirs, plain_models):
    name = "A"
    config, tensors = plain_models[name]
    prompt = tt.random_tokens(77, 9, CONFIGS[name][0]["vocab_size"])
    cmd = [sys.executable, os.path.join(ROOT, "bin", "liyab-cli"), "-m", model_dirs[name], "-p",
           ",".join(map(str, prompt)), "-n", "12", "--temp", "0", "--dtype", "float32", "--json"]
    p = subprocess.run(cmd, capture_output=True, text=True, timeout=600)
    assert p.returncode == 0, p.stderr[-3000:]
    lines = [json.loads(l) for l in p.stdout.splitlines() if l.startswith("{")]
    assert "load_ms" in lines[0]
    turn = lines[1]
    assert turn["prompt_tokens"] == 9 and turn["generated_tokens"] == len(turn["tokens"])
    expect = plain.generate_greedy(config, tensors, prompt, 12)
    eos = config.get("eos_token_id")
    assert turn["tokens"] == expect[:len(turn["tokens"])] and (len(turn["tokens"]) == 12 or turn["tokens"][-1] == eos)
    assert "decode:" in p.stderr and "prompt: 9 tokens" in p.stderr
    assert "phases_ms" not in turn
    # per-phase device times behind a flag; the tokens are the same
    p2 = subprocess.run(cmd + ["--phases"], capture_output=True, text=True, timeout=600)
    assert p2.returncode == 0, p2.stderr[-3000:]
    turn2 = [json.loads(l) for l in p2.stdout.splitlines() if l.startswith("{")][1]
    assert turn2["tokens"] == turn["tokens"]
    assert set(turn2["phases_ms"]) == {"embed", "attention", "dense_ffn", "lm_head"}
    assert all(v > 0 for v in turn2["phases_ms"].values()) and "phases (ms/token)" in p2.stderr


# ---------------------------------------------------------------------------
# real widths
# ---------------------------------------------------------------------------
SIZES = {
    # GPT-2 small's sizes, all 12 layers
    "small": dict(n_layer=12, n_embd=768, n_head=12, n_inner=3072, vocab_size=50257, n_positions=1024, seed=10,
                  lens=[300, 77, 130]),
    # GPT-2 XL's layer sizes (width 1600, 25 heads, feed-forward 6400), two layers, a small vocabulary
    "xl_layers": dict(n_layer=2, n_embd=1600, n_head=25, n_inner=6400, vocab_size=3001, n_positions=512, seed=30,
                      lens=[200, 33, 90]),
    # GPT-2 medium's and large's layer sizes (widths 1,024 and 1,280: 16 and 20 units of 64 to a row), two layers each
    "medium_layers": dict(n_layer=2, n_embd=1024, n_head=16, n_inner=4096, vocab_size=2999, n_positions=512, seed=20,
                          lens=[150, 40, 9]),
    "large_layers": dict(n_layer=2, n_embd=1280, n_head=20, n_inner=5120, vocab_size=3003, n_positions=512, seed=25,
                         lens=[170, 35, 64]),
    # three heads of 48 in a width of 144, a vocabulary that is no multiple of anything
    "odd": dict(n_layer=2, n_embd=144, n_head=3, n_inner=200, vocab_size=777, n_positions=640, seed=5,
                lens=[600, 45, 170]),
}


@pytest.fixture(scope="module")
def sized_models(tmp_path_factory):
    """{name: (folder, requests, {dtype: plain logits})}, each made on first use."""
    made = {}

    def get(name):
        if name not in made:
            from liyab_amd.weights import write_random_model

            s = SIZES[name]
            cfg = {"architectures": ["GPT2LMHeadModel"], "layer_norm_epsilon": 1e-5, "activation_function": "gelu_new",
                   **{k: s[k] for k in ("n_layer", "n_embd", "n_head", "n_inner", "vocab_size", "n_positions")}}
            d = str(tmp_path_factory.mktemp(f"sized_{name}"))
            write_random_model(d, cfg, s["seed"])
            config, tensors = plain.read_model(d)
            reqs = {f"{name}{i}": tt.random_tokens(s["seed"] + 1 + i, n, s["vocab_size"]) for i, n in enumerate(s["lens"])}
            refs = {"float32": {rid: plain.forward(config, tensors, t) for rid, t in reqs.items()}}
            rounded = plain.round_weights_to_bf16(tensors)
            refs["bfloat16"] = {rid: plain.forward(config, rounded, t) for rid, t in reqs.items()}
            made[name] = (d, reqs, refs)
        return made[name]

    return get


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(SIZES))
def test_real_widths_whole_and_mixed(name, dtype, sized_models):
    """GPT-2 small's full sizes, medium's, large's and XL's layer sizes and an odd geometry: whole prompts and a
    mixed schedule with pages used again, against the plain implementation."""
    d, reqs, refs = sized_models(name)
    for label, steps in (("whole", tt.schedule_whole(reqs)), ("mixed", tt.schedule_mixed(reqs, seed=1, decode_tail=6))):
        core = make_core(d, dtype, tt.max_live_tokens(steps))
        got = tt.run_schedule(core, steps)
        tt.check_against_plain(got, reqs, refs[dtype], TOL[dtype], f"{name} {label} {dtype}", family=f"sizes:{name}")
        core.manager.check()
        del core


@pytest.mark.parametrize("dtype", DTYPES)
def test_overlapped_steps_give_the_same_tokens(dtype, model_dirs):
    """The engine launches the next step before it has read this step's tokens; with or without
    that overlap, greedy or sampled, stopping at an end token or not, the tokens are the same."""
    from liyab_amd import Engine, SamplingParams

    name = "B"
    V = CONFIGS[name][0]["vocab_size"]
    prompts = [tt.random_tokens(80 + i, n, V) for i, n in enumerate([1, 13, 64, 100, 5, 30])]
    for sp in (SamplingParams(temperature=0.0, max_tokens=40), SamplingParams(temperature=0.9, top_k=50, top_p=0.9, seed=9, max_tokens=40)):
        results = {}
        for overlap in (False, True):
            engine = Engine(model_dirs[name], dtype=dtype, page_size=16, num_pages=24, max_num_seqs=4, max_batched_tokens=48,
                            prefill_chunk=32, overlap=overlap)
            engine.stop_at_eos = False
            free = engine.generate(prompts, sp)
            # an end token that request 2 draws in the middle: it and others must stop there
            eos = free[2].tokens[11]
            engine.scheduler.eos_token_id = eos
            engine.stop_at_eos = True
            stopped = engine.generate(prompts, sp)
            for a, b in zip(free, stopped):
                cut = a.tokens.index(eos) + 1 if eos in a.tokens else len(a.tokens)
                assert b.tokens == a.tokens[:cut]
                assert b.finish_reason == ("stop" if eos in a.tokens else a.finish_reason)
            results[overlap] = ([r.tokens for r in free], [r.tokens for r in stopped])
            assert engine.core.manager.pages_in_use() == 0
            engine.core.manager.check()
        assert results[False] == results[True]


# ---------------------------------------------------------------------------
# drawn geometries
# ---------------------------------------------------------------------------
def drawn_config(seed):
    """A GPT-2 configuration drawn from the seed: any number of heads, head sizes in steps of
    16 up to 256, a feed-forward width and a vocabulary that are multiples of nothing."""
    rng = np.random.default_rng(1000 + seed)
    hd = int(rng.choice([16, 32, 48, 64, 80, 96, 112, 128, 144, 192, 256]))
    n_head = int(rng.integers(1, 8 if hd <= 64 else 4))
    return {"architectures": ["GPT2LMHeadModel"], "n_layer": int(rng.integers(1, 4)), "n_embd": hd * n_head, "n_head": n_head,
            "n_inner": int(rng.integers(17, 400)), "vocab_size": int(rng.integers(50, 1500)),
            "n_positions": int(rng.integers(150, 330)), "layer_norm_epsilon": float(rng.choice([1e-5, 1e-6, 3e-4])),
            "activation_function": str(rng.choice(["gelu_new", "gelu"])),
            "scale_attn_by_inverse_layer_idx": bool(rng.integers(0, 2)), "scale_attn_weights": bool(rng.integers(0, 4) > 0)}


@pytest.mark.parametrize("seed", range(10))
def test_drawn_geometries_whole_and_mixed(seed, tmp_path):
    """Ten drawn configurations, each whole and in a mixed schedule, in both precisions: a size
    the kernels mishandle shows as a wrong logit (or a refusal), never passes silently."""
    from liyab_amd.weights import write_random_model

    cfg = drawn_config(seed)
    write_random_model(str(tmp_path), cfg, 200 + seed)
    config, tensors = plain.read_model(str(tmp_path))
    P, V = cfg["n_positions"], cfg["vocab_size"]
    reqs = {f"g{i}": tt.random_tokens(300 + 10 * seed + i, n, V) for i, n in enumerate([P, 41, 1 + seed, 130])}
    for dtype in DTYPES:
        weights = tensors if dtype == "float32" else plain.round_weights_to_bf16(tensors)
        refs = {rid: plain.forward(config, weights, t) for rid, t in reqs.items()}
        for label, steps in (("whole", tt.schedule_whole(reqs)), ("mixed", tt.schedule_mixed(reqs, seed=seed, decode_tail=5))):
            core = make_core(str(tmp_path), dtype, tt.max_live_tokens(steps))
            got = tt.run_schedule(core, steps)
            tt.check_against_plain(got, reqs, refs, TOL[dtype], f"{cfg} {label} {dtype}", family="drawn")
            core.manager.check()
            del core


def test_random_workloads_through_the_scheduler(tmp_path):
    """Sixty workloads drawn from a seed, each with its own budgets (positions a page, pages, live
    requests, tokens a step, tokens a portion, graphs on or off), most of them too tight for the
    requests at hand, so that prompts are cut, pages run out and requests are preempted and taken up
    again: in float32 every greedy token is the plain implementation's choice, every request gets
    its number of tokens, and no page is lost. (The preemptions are counted: the draw must bring some.)"""
    from liyab_amd import Engine, SamplingParams
    from liyab_amd.weights import write_random_model

    cfg = dict(drawn_config(2), n_positions=160)
    write_random_model(str(tmp_path), cfg, 77)
    config, tensors = plain.read_model(str(tmp_path))
    preemptions = 0
    for seed in range(60):
        rng = np.random.default_rng(5000 + seed)
        prompts = [tt.random_tokens(seed * 100 + i, int(rng.integers(1, 90)), cfg["vocab_size"]) for i in range(int(rng.integers(1, 9)))]
        n_new = int(rng.integers(1, 40))
        page = int(rng.choice([4, 8, 16]))
        need_one = -(-(max(len(p) for p in prompts) + n_new) // page)
        kw = dict(page_size=page, num_pages=int(rng.integers(need_one, need_one * 4 + 2)), max_num_seqs=int(rng.integers(1, 7)),
                  max_batched_tokens=int(rng.integers(8, 200)), prefill_chunk=int(rng.integers(2, 64)), use_graphs=bool(rng.integers(0, 2)))
        engine = Engine(str(tmp_path), dtype="float32", **kw)
        engine.stop_at_eos = False
        results = engine.generate(prompts, SamplingParams(temperature=0.0, max_tokens=n_new))
        for i, (prompt, res) in enumerate(zip(prompts, results)):
            assert len(res.tokens) == n_new, (seed, kw, i)
            ref = plain.forward(config, tensors, prompt + res.tokens[:-1])
            for j, t in enumerate(res.tokens):
                row = ref[len(prompt) - 1 + j]
                assert row[t] >= row.max() - 1e-5 * np.abs(row).max(), (seed, kw, i, j, t, int(np.argmax(row)))
        engine.core.manager.check()
        assert all(engine.core.manager.pages_in_use(g.index) == 0 for g in engine.core.manager.groups)
        preemptions += engine.scheduler.stats.preemptions
    assert preemptions > 20
