"""Paths of the engine that a plain run of prompts does not reach (needs the GPU): a pool so
small that requests are preempted and recomputed, HIP graphs replayed and compared with eager
runs of the same steps, geometries that take the kernels' fallbacks in bfloat16, a head of its
own (untied), and sizes refused when a model is built."""

import numpy as np
import pytest

import plain_gpt2 as plain
import trace_tools as tt
from conftest import CONFIGS, TOL

pytestmark = pytest.mark.gpu

DTYPES = ["float32", "bfloat16"]


def _near_argmax(ref_row, token, tol):
    ref_row = np.asarray(ref_row, dtype=np.float64)
    return ref_row[token] >= ref_row.max() - tol * np.abs(ref_row).max()


# ---------------------------------------------------------------------------
# preemption and recomputation on the device
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("overlap", [False, True])
@pytest.mark.parametrize("mode", DTYPES + ["bfloat16 batch-invariant"])
def test_preempted_requests_are_recomputed_to_the_same_tokens(mode, overlap, model_dirs, plain_models):
    """Three prompts of 30 tokens that each grow to 74 positions (5 pages of 16) in a pool of 8
    pages: they cannot all stay, so the latest admitted is preempted, its pages go to the others
    and it is recomputed from its prompt plus what it had generated, through pages other
    requests have used. Greedy and seeded: the tokens are those of each request alone (in
    32-bit also the plain implementation's), whatever was preempted when; in bfloat16 that holds
    bit for bit in the batch-invariant mode, and within the tolerance of the plain choice otherwise."""
    from liyab_amd import Engine, SamplingParams

    dtype, invariant = mode.split()[0], "invariant" in mode
    name = "B"
    cfg, _ = CONFIGS[name]
    config, tensors = plain_models[name]
    weights = tensors if dtype == "float32" else plain.round_weights_to_bf16(tensors)
    V = cfg["vocab_size"]
    prompts = [tt.random_tokens(900 + i, 30, V) for i in range(3)]
    for sp in (SamplingParams(temperature=0.0, max_tokens=45),
               SamplingParams(temperature=0.8, top_k=0, top_p=1.0, seed=4, max_tokens=45)):
        tight = Engine(model_dirs[name], dtype=dtype, page_size=16, num_pages=8, max_num_seqs=3, max_batched_tokens=64,
                       prefill_chunk=32, overlap=overlap, batch_invariant=invariant)
        tight.stop_at_eos = False
        for c in tight.core.storage.layers.values():  # free pages hold NaN
            for t in c.rows.values():
                t.fill_(float("nan"))
        together = tight.generate(prompts, sp)
        stats = tight.scheduler.stats
        assert stats.preemptions >= 1, "the pool held every request: nothing was preempted"
        assert sum(r.stats.preemptions for r in together) == stats.preemptions
        assert tight.core.manager.pages_in_use() == 0
        tight.core.manager.check()
        assert tight.core.step_fn.graph_replays > 0
        roomy = Engine(model_dirs[name], dtype=dtype, page_size=16, num_pages=64, max_num_seqs=3, max_batched_tokens=64,
                       prefill_chunk=32, overlap=overlap, batch_invariant=invariant)
        roomy.stop_at_eos = False
        alone = [roomy.generate(p, sp) for p in prompts]
        assert roomy.scheduler.stats.preemptions == 0
        for prompt, a, b in zip(prompts, together, alone):
            assert len(a.tokens) == 45 and a.finish_reason == "length"
            if dtype == "float32" or invariant:
                assert a.tokens == b.tokens
                if sp.temperature == 0.0 and dtype == "float32":
                    assert a.tokens == plain.generate_greedy(config, tensors, prompt, 45)
            if dtype == "bfloat16" and sp.temperature == 0.0:
                # bfloat16: each token is the plain implementation's choice given the tokens before it,
                # within the tolerance (a recomputed prompt goes through other kernels than single tokens)
                ref = plain.forward(config, weights, prompt + a.tokens[:-1])
                for i, t in enumerate(a.tokens):
                    assert _near_argmax(ref[len(prompt) - 1 + i], t, TOL[dtype]), f"token {i}"


# ---------------------------------------------------------------------------
# HIP graphs: replays happen, and give what eager runs give
# ---------------------------------------------------------------------------
def _graph_schedule(V, P):
    """Steps that bring the same shapes again and again with different contents: a decode shape
    (two requests, one token each) many times, across a context bucket's edge (256); and a
    mixed shape of 500 tokens cut (300, 200) and (270, 230), which fall into the same tiles and
    the same bucket, five times and more."""
    assert P >= 600
    steps = []
    a = tt.random_tokens(1, 300, V)
    b = tt.random_tokens(2, 300, V)
    # two requests that decode from 250 to 262: the bucket changes from 256 to 512 on the way
    steps.append({"entries": [("a", a[:250], [249]), ("b", b[:250], [0, 249])], "end": []})
    for i in range(250, 262):
        steps.append({"entries": [("a", a[i:i + 1], [0]), ("b", b[i:i + 1], [0])], "end": ["a", "b"] if i == 261 else []})
    # the mixed shape, each time with other tokens and another cut
    for i in range(7):
        x = tt.random_tokens(10 + i, 300, V)
        y = tt.random_tokens(30 + i, 300, V)
        nx, ny = (300, 200) if i % 2 == 0 else (270, 230)
        steps.append({"entries": [(f"x{i}", x[:nx], [0, nx - 1]), (f"y{i}", y[:ny], [ny - 1])], "end": [f"x{i}", f"y{i}"]})
    # a decode shape of three requests beside, so that a small table of graphs has to drop one
    c = tt.random_tokens(3, 40, V)
    steps.append({"entries": [("a2", a[:20], []), ("b2", b[:20], []), ("c2", c[:20], [])], "end": []})
    for i in range(20, 26):
        steps.append({"entries": [("a2", a[i:i + 1], [0]), ("b2", b[i:i + 1], [0]), ("c2", c[i:i + 1], [0])], "end": []})
    for i in range(26, 32):  # back to two: its graph may have been dropped meanwhile, and is captured again
        steps.append({"entries": [("a2", a[i:i + 1], [0]), ("b2", b[i:i + 1], [0])], "end": []})
    steps[-1]["end"] = ["a2", "b2", "c2"]
    return steps


def _run_steps(core, steps):
    from liyab_amd.engine import StepItem

    out = []
    for st in steps:
        items = []
        for rid, toks, want in st["entries"]:
            if not core.is_open(rid):
                core.open(rid)
            items.append(StepItem(rid, toks, want))
        logits = core.step(items)
        out.append(None if logits is None else logits.float().cpu().numpy().copy())
        for rid in st["end"]:
            core.close(rid)
    return out


@pytest.mark.parametrize("max_graphs", [256, 2])
@pytest.mark.parametrize("dtype", DTYPES)
def test_replayed_graphs_give_the_eager_logits(dtype, max_graphs, model_dirs):
    """The same steps through an engine that captures and replays HIP graphs and through one that
    launches every kernel itself: the same bits at every step. Shapes recur with other contents
    (other tokens, other cuts into requests, a context past a bucket's edge), so a kernel argument
    that a graph had baked in where it should have come from the step's metadata would show.
    With room for two graphs only, shapes are dropped and captured again in between."""
    from liyab_amd.engine import EngineCore

    name = "C"
    cfg, _ = CONFIGS[name]
    steps = _graph_schedule(cfg["vocab_size"], cfg["n_positions"])
    eager = EngineCore(model_dirs[name], dtype=dtype, page_size=16, max_tokens=2048, max_requests=8, use_graphs=False)
    want = _run_steps(eager, steps)
    assert eager.step_fn.graph_replays == 0
    graphs = EngineCore(model_dirs[name], dtype=dtype, page_size=16, max_tokens=2048, max_requests=8, use_graphs=True)
    graphs.step_fn.max_graphs = max_graphs
    got = _run_steps(graphs, steps)
    fn = graphs.step_fn
    captured = [k for k, v in fn._graphs.items() if isinstance(v, tuple)]
    assert fn.graph_replays >= (15 if max_graphs > 2 else 8), fn.graph_replays
    if max_graphs > 2:
        modes = {term[1][0] for k in captured for term in k[3:] if term[0] == "attention"}
        assert modes == {"decode", "prefill"}, captured
    else:
        assert len(fn._graphs) <= 2
    for i, (g, w) in enumerate(zip(got, want)):
        assert (g is None) == (w is None)
        if g is not None:
            assert np.array_equal(g, w), f"step {i} ({[(r, len(t)) for r, t, _ in steps[i]['entries']]}): replayed and eager logits differ"
    graphs.manager.check()
    assert graphs.manager.pages_in_use() == 0


@pytest.mark.parametrize("dtype", DTYPES)
def test_prompts_of_one_padded_size_share_a_graph(dtype, model_dirs):
    """Steps in which a request brings several tokens are padded to sizes that recur (rows behind
    their tokens that belong to no request): prompts of 33 to 48 tokens are one shape, launched
    kernel by kernel three times, then captured once and replayed. Logits have the bits of an engine
    that neither pads nor captures, also when everything the padding rows might leave behind (the
    workspace's buffers) is filled with NaN between the steps, and with pages that are used again."""
    import torch

    from liyab_amd.engine import EngineCore, StepItem
    from liyab_amd.engine.step import padded_rows

    assert [padded_rows(n) for n in (2, 16, 17, 33, 48, 64, 65, 500, 1024, 1025)] == [16, 16, 32, 48, 48, 64, 128, 512, 1024, 1152]
    name = "C"
    cfg, _ = CONFIGS[name]
    rng = np.random.default_rng(5)
    plain_core = EngineCore(model_dirs[name], dtype=dtype, page_size=16, max_tokens=64, max_requests=2, use_graphs=False)
    core = EngineCore(model_dirs[name], dtype=dtype, page_size=16, max_tokens=64, max_requests=2, use_graphs=True)
    assert core.step_fn.pads_rows and not plain_core.step_fn.pads_rows
    lengths = [37, 45, 40, 33, 48, 41, 47, 34]
    for i, n in enumerate(lengths):
        toks = rng.integers(0, cfg["vocab_size"], n).tolist()
        want = [0, n // 2, n - 1]
        out = []
        for c in (plain_core, core):
            c.open("r")
            before = c.step_fn.graph_replays
            first = c.step([StepItem("r", toks, want)]).float().cpu().numpy().copy()
            replayed = c.step_fn.graph_replays > before
            after = c.step([StepItem("r", [toks[0]], [0])]).float().cpu().numpy().copy()  # a decoded token reads the portion's keys
            c.close("r")
            out.append((first, after))
        assert np.array_equal(out[0][0], out[1][0]) and np.array_equal(out[0][1], out[1][1]), f"prompt {i} of {n} tokens"
        assert np.isfinite(out[1][0]).all()
        # three sights launched kernel by kernel, then the capture (once more if a buffer of the workspace grew under it)
        assert not (replayed and i < 3) and (replayed or i < 5), f"prompt {i}: replayed {replayed}"
        for buf in core.step_fn.workspace._bufs.values():
            if buf.is_floating_point():
                buf.fill_(float("nan"))
        torch.cuda.synchronize()
    fn = core.step_fn
    prefill_graphs = [k for k, v in fn._graphs.items() if isinstance(v, tuple) and k[0] == 48]
    assert len(prefill_graphs) == 1, list(fn._graphs)
    assert fn.graph_replays >= len(lengths), fn.graph_replays
    core.manager.check()
    assert core.manager.pages_in_use() == 0


# ---------------------------------------------------------------------------
# geometries that take the kernels' fallbacks in bfloat16; a head of its own
# ---------------------------------------------------------------------------
FALLBACKS = {
    # width 60 = 3 heads of 20: no multiple of 8, so in bfloat16 neither the matrix-core products nor
    # the paged QKV epilogue nor the fast attention take it (plain product + kv_write + plain attention)
    "w60_h20": dict(n_layer=2, n_embd=60, n_head=3, n_inner=100, vocab_size=333, n_positions=200),
    # width 44 = 4 heads of 11
    "w44_h11": dict(n_layer=1, n_embd=44, n_head=4, n_inner=50, vocab_size=97, n_positions=160,
                    activation_function="gelu", scale_attn_by_inverse_layer_idx=True),
    # heads of 40 (8 x odd): matrix cores for the products, the decode kernel, no tiled prefill attention
    "w120_h40": dict(n_layer=2, n_embd=120, n_head=3, n_inner=90, vocab_size=500, n_positions=300),
    # heads of 24 in a width of 72, an untied head and eps 1e-6
    "w72_h24_untied": dict(n_layer=2, n_embd=72, n_head=3, n_inner=64, vocab_size=211, n_positions=180,
                           tie_word_embeddings=False, layer_norm_epsilon=1e-6),
    # an untied head at sizes every fast kernel takes
    "w64_untied": dict(n_layer=2, n_embd=64, n_head=2, n_inner=256, vocab_size=1031, n_positions=256,
                       tie_word_embeddings=False),
}


@pytest.mark.parametrize("name", list(FALLBACKS))
def test_fallback_geometries_whole_and_mixed(name, tmp_path):
    from liyab_amd.engine import EngineCore
    from liyab_amd.weights import write_random_model

    cfg = {"architectures": ["GPT2LMHeadModel"], "layer_norm_epsilon": 1e-5, "activation_function": "gelu_new", **FALLBACKS[name]}
    seed = 700 + list(FALLBACKS).index(name)
    write_random_model(str(tmp_path), cfg, seed)
    config, tensors = plain.read_model(str(tmp_path))
    if not cfg.get("tie_word_embeddings", True):
        assert "lm_head.weight" in tensors and not np.array_equal(tensors["lm_head.weight"], tensors["wte.weight"])
    P, V = cfg["n_positions"], cfg["vocab_size"]
    reqs = {f"f{i}": tt.random_tokens(seed * 10 + i, n, V) for i, n in enumerate([P, 37, 3, 101])}
    for dtype in DTYPES:
        weights = tensors if dtype == "float32" else plain.round_weights_to_bf16(tensors)
        refs = {rid: plain.forward(config, weights, t) for rid, t in reqs.items()}
        for label, steps in (("whole", tt.schedule_whole(reqs)), ("mixed", tt.schedule_mixed(reqs, seed=seed, decode_tail=7)),
                             ("portions", tt.schedule_portions(reqs, (5, 2, 17, 3, 48, 2)))):
            core = EngineCore(str(tmp_path), dtype=dtype, page_size=16, max_tokens=tt.max_live_tokens(steps), max_requests=8)
            for c in core.storage.layers.values():
                for t in c.rows.values():
                    t.fill_(float("nan"))
            got = tt.run_schedule(core, steps)
            tt.check_against_plain(got, reqs, refs, TOL[dtype], f"{name} {label} {dtype}", family=f"fallback:{name}")
            core.manager.check()
            assert core.manager.pages_in_use() == 0
            del core


def test_untied_head_is_the_heads_own_matrix(tmp_path):
    """With tie_word_embeddings false the logits come from lm_head.weight: they equal the plain
    implementation's with its own head and are far from what the embedding table as head gives."""
    from liyab_amd.engine import EngineCore, StepItem
    from liyab_amd.weights import write_random_model

    cfg = {"architectures": ["GPT2LMHeadModel"], **FALLBACKS["w64_untied"]}
    write_random_model(str(tmp_path), cfg, 5)
    config, tensors = plain.read_model(str(tmp_path))
    toks = tt.random_tokens(8, 50, cfg["vocab_size"])
    core = EngineCore(str(tmp_path), dtype="float32", page_size=16, max_tokens=64)
    core.open("r")
    got = core.step([StepItem("r", toks, list(range(50)))]).cpu().numpy()
    assert tt.rel_err(got, plain.forward(config, tensors, toks)) <= TOL["float32"]
    tied = dict(config, tie_word_embeddings=True)
    assert tt.rel_err(got, plain.forward(tied, tensors, toks)) > 1e-2  # the embedding table is not the head


def test_head_sizes_the_kernels_cannot_take_are_refused_at_load(tmp_path):
    """One head of 272: no attention kernel takes it, and the model says so when it is built
    (from a folder, and already when the random-weights mode builds it), not at its first step."""
    import json

    import torch

    from liyab_amd import Unsupported
    from liyab_amd.engine import EngineCore
    from liyab_amd.weights import write_random_model, write_safetensors

    d, F, V, P = 272, 16, 20, 16
    cfg = {"architectures": ["GPT2LMHeadModel"], "n_layer": 1, "n_embd": d, "n_head": 1, "n_inner": F, "vocab_size": V,
           "n_positions": P}
    with pytest.raises(Unsupported, match="272"):
        write_random_model(str(tmp_path / "drawn"), cfg, 1)
    shapes = {"wte.weight": (V, d), "wpe.weight": (P, d), "ln_f.weight": (d,), "ln_f.bias": (d,), "h.0.ln_1.weight": (d,),
              "h.0.ln_1.bias": (d,), "h.0.ln_2.weight": (d,), "h.0.ln_2.bias": (d,), "h.0.attn.c_attn.weight": (d, 3 * d),
              "h.0.attn.c_attn.bias": (3 * d,), "h.0.attn.c_proj.weight": (d, d), "h.0.attn.c_proj.bias": (d,),
              "h.0.mlp.c_fc.weight": (d, F), "h.0.mlp.c_fc.bias": (F,), "h.0.mlp.c_proj.weight": (F, d), "h.0.mlp.c_proj.bias": (d,)}
    folder = tmp_path / "written"
    folder.mkdir()
    (folder / "config.json").write_text(json.dumps(cfg))
    write_safetensors(str(folder / "model.safetensors"), {k: torch.zeros(s) for k, s in shapes.items()}, {})
    with pytest.raises(Unsupported, match="272"):
        EngineCore(str(folder), dtype="float32", page_size=16, max_tokens=64)


# ---------------------------------------------------------------------------
# layers of one kind run from one recorded list of launches
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("use_graphs", [False, True])
@pytest.mark.parametrize("dtype", DTYPES)
def test_layers_run_from_a_recorded_list_give_the_bits_of_their_own_python(dtype, use_graphs, tmp_path):
    """Five layers of one kind: the second layer's launches are written down as it runs and the
    third to fifth run from that list with their own weights and pages in place of the second's
    (the first finds the stream whole, the others split, so it is a kind of its own in
    bfloat16). Whole prompts, portions, mixed batches and single tokens, eager and under graphs:
    the logits have the bits of the same engine with every layer run through its Python, and are
    the plain implementation's."""
    from liyab_amd.engine import EngineCore
    from liyab_amd.weights import write_random_model

    cfg = {"architectures": ["GPT2LMHeadModel"], "n_layer": 5, "n_embd": 128, "n_head": 4, "n_inner": 320, "vocab_size": 700,
           "n_positions": 300, "layer_norm_epsilon": 1e-5, "activation_function": "gelu_new"}
    write_random_model(str(tmp_path), cfg, 41)
    config, tensors = plain.read_model(str(tmp_path))
    weights = tensors if dtype == "float32" else plain.round_weights_to_bf16(tensors)
    reqs = {f"l{i}": tt.random_tokens(70 + i, n, 700) for i, n in enumerate([150, 33, 9, 70, 260])}
    refs = {rid: plain.forward(config, weights, t) for rid, t in reqs.items()}
    for label, steps in (("whole", tt.schedule_whole(reqs)), ("mixed", tt.schedule_mixed(reqs, seed=6, decode_tail=8)),
                         ("bulk+tail", tt.schedule_bulk_tail(reqs, tail=9))):
        runs = {}
        for replay in (True, False):
            core = EngineCore(str(tmp_path), dtype=dtype, page_size=16, max_tokens=tt.max_live_tokens(steps), max_requests=8,
                              use_graphs=use_graphs)
            core.model.replay_layers = replay
            runs[replay] = tt.run_schedule(core, steps)
            if replay:
                assert core.model.replayed_layers >= 3 * (len(steps) - core.step_fn.graph_replays) - 3, "the layers ran through their Python"
            else:
                assert core.model.replayed_layers == 0
            core.manager.check()
            del core
        for rid, toks in reqs.items():
            for p in range(len(toks)):
                assert np.array_equal(runs[True][rid][p], runs[False][rid][p]), f"{label}: request {rid} position {p}: other bits from the recorded list"
        tt.check_against_plain(runs[True], reqs, refs, TOL[dtype], f"recorded layers {label} {dtype}", family="sizes:odd")


def test_layers_with_constants_of_their_own_are_not_run_from_anothers_list(model_dirs):
    """Configuration B scales attention by 1 / (layer + 1): a constant that differs from layer to
    layer makes every layer a kind of its own, and each runs through its own Python."""
    from liyab_amd.engine import EngineCore

    for name, replays in (("A", True), ("B", False)):
        core = EngineCore(model_dirs[name], dtype="float32", page_size=16, max_tokens=256, max_requests=2, use_graphs=False)
        kinds = core.model._layer_kind
        assert (kinds[0] == kinds[1]) == replays
        core.open("r")
        core.step([tt_item("r", [1, 2, 3, 4, 5], [4])])
        assert (core.model.replayed_layers > 0) == replays


def tt_item(rid, tokens, want):
    from liyab_amd.engine import StepItem

    return StepItem(rid, tokens, want)


def test_a_malformed_list_of_launches_is_refused_before_anything_runs():
    from liyab_amd.kernels import lib

    lib.load()
    index, kinds = lib._encoders("liyab_fill")
    assert index >= 0 and len(kinds) == 5
    for words, what in (([index, 5, 0, 4, 0, 0], "cut short"), ([9999, 0, 0], "unknown launcher"), ([index, 4, 0, 4, 0, 0, 0], "takes 5 arguments"),
                        ([index, 5, lib.BLOCK_ARG, 4, 0, 0, 0, 0], "parameter block")):
        with pytest.raises(Exception, match=what):
            lib.replay(np.array(words, dtype=np.uint64))
    product, kinds = lib._encoders("liyab_gemm_mfma")
    assert product >= 0 and kinds[7] == "block" and len(kinds) == 9
    with pytest.raises(Exception, match="shorter than the launchers read"):  # one word where the epilogue's parameters stand
        lib.replay(np.array([product, 9, 0, 0, 0, 0, 0, 0, 0, lib.BLOCK_ARG, 0, 1, 0], dtype=np.uint64))
    lib.replay(np.array([], dtype=np.uint64))


# ---------------------------------------------------------------------------
# bfloat16 replies that do not depend on the batch
# ---------------------------------------------------------------------------
@pytest.fixture(scope="module")
def small_widths_model(tmp_path_factory):
    """GPT-2 small's widths and vocabulary, three layers."""
    from liyab_amd.weights import write_random_model

    cfg = {"architectures": ["GPT2LMHeadModel"], "n_layer": 3, "n_embd": 768, "n_head": 12, "n_inner": 3072, "vocab_size": 50257,
           "n_positions": 1024, "layer_norm_epsilon": 1e-5, "activation_function": "gelu_new"}
    d = str(tmp_path_factory.mktemp("small_widths"))
    write_random_model(d, cfg, 10, dtype="bfloat16")
    return d, cfg


def test_batch_invariant_logits_have_the_same_bits_alone_and_together(small_widths_model):
    """With batch_invariant the bfloat16 logits of a position are the same bits however the
    tokens are cut into steps and whatever else a step holds: whole prompts, the last tokens
    one by one, portions of changing size, and mixed batches of up to four requests."""
    from liyab_amd.engine import EngineCore

    d, cfg = small_widths_model
    V = cfg["vocab_size"]
    # (the request of 950 tokens: its whole prompt walks four splits of 256 keys in one workgroup a
    # token and head, its last tokens are launched in splits side by side)
    reqs = {f"i{i}": tt.random_tokens(500 + i, n, V) for i, n in enumerate([150, 33, 9, 70, 260, 950])}
    runs = {}
    for label, steps in (("whole", tt.schedule_whole(reqs)), ("tail", tt.schedule_bulk_tail(reqs, tail=12)),
                         ("portions", tt.schedule_portions(reqs, (5, 2, 17, 3, 48, 2, 31, 7))),
                         ("mixed", tt.schedule_mixed(reqs, seed=4, decode_tail=10))):
        core = EngineCore(d, dtype="bfloat16", page_size=16, max_tokens=tt.max_live_tokens(steps), max_requests=8,
                          batch_invariant=True)
        runs[label] = tt.run_schedule(core, steps)
        assert core.step_fn.graph_replays > 0 or label == "whole"
        del core
    for label in ("tail", "portions", "mixed"):
        for rid, toks in reqs.items():
            for p in range(len(toks)):
                assert np.array_equal(runs[label][rid][p], runs["whole"][rid][p]), \
                    f"{label}: request {rid} position {p} differs from its logits alone and whole"
    # the step-shaped kernels of the default mode agree with these within the tolerance, not bit for bit
    steps = tt.schedule_mixed(reqs, seed=4, decode_tail=10)
    core = EngineCore(d, dtype="bfloat16", page_size=16, max_tokens=tt.max_live_tokens(steps), max_requests=8)
    fast = tt.run_schedule(core, steps)
    worst = max(tt.rel_err(fast[rid][p], runs["whole"][rid][p]) for rid, toks in reqs.items() for p in range(len(toks)))
    assert 0 < worst <= TOL["bfloat16"]


def test_float32_logits_have_the_same_bits_whole_and_token_by_token(small_widths_model):
    """The 32-bit path at GPT-2 small's widths, a request of 950 tokens: whole (one workgroup a
    token and head walks four splits of 256 keys), in portions, and its last tokens one by one
    (the splits launched side by side) give the same bits, and the plain implementation's
    logits within the 32-bit tolerance."""
    from liyab_amd.engine import EngineCore

    d, cfg = small_widths_model
    config, tensors = plain.read_model(d)
    reqs = {"f0": tt.random_tokens(700, 950, cfg["vocab_size"]), "f1": tt.random_tokens(701, 40, cfg["vocab_size"])}
    sparse = lambda steps: [dict(s, entries=[(r, t, w[-4:]) for r, t, w in s["entries"]]) for s in steps]  # noqa: E731
    runs = {}
    for label, steps in (("whole", sparse(tt.schedule_whole(reqs))), ("tail", sparse(tt.schedule_bulk_tail(reqs, tail=6))),
                         ("mixed", sparse(tt.schedule_mixed(reqs, seed=1, decode_tail=5, portions=(300, 9, 48))))):
        core = EngineCore(d, dtype="float32", page_size=16, max_tokens=tt.max_live_tokens(steps), max_requests=4)
        runs[label] = tt.run_schedule(core, steps)
        del core
    refs = {rid: plain.forward(config, tensors, t) for rid, t in reqs.items()}
    tt.check_against_plain(runs["whole"], reqs, refs, TOL["float32"], "float32, 950 tokens whole", family="sizes:small")
    for label in ("tail", "mixed"):
        tt.check_against_plain(runs[label], reqs, refs, TOL["float32"], f"float32, 950 tokens {label}", family="sizes:small")
        for rid in reqs:
            for p in set(runs[label][rid]) & set(runs["whole"][rid]):
                assert np.array_equal(runs[label][rid][p], runs["whole"][rid][p]), f"{label}: request {rid} position {p}: other bits than whole"
    assert set(runs["tail"]["f0"]) & set(runs["whole"]["f0"]) >= {946, 949}


@pytest.mark.parametrize("overlap", [False, True])
def test_batch_invariant_replies_are_the_same_alone_and_among_eight(small_widths_model, overlap):
    """Greedy and seeded replies in bfloat16 at GPT-2 small's widths: the same tokens for a
    request alone and among eight, with random weights, whose logits lie close together."""
    from liyab_amd import Engine, SamplingParams

    d, cfg = small_widths_model
    prompts = [tt.random_tokens(600 + i, n, cfg["vocab_size"]) for i, n in enumerate([40, 7, 120, 64, 1, 90, 33, 15])]
    engine = Engine(d, dtype="bfloat16", page_size=16, max_num_seqs=8, max_batched_tokens=256, prefill_chunk=64,
                    batch_invariant=True, overlap=overlap)
    engine.stop_at_eos = False
    for sp in (SamplingParams(temperature=0.0, max_tokens=32),
               SamplingParams(temperature=0.8, top_k=40, top_p=0.95, seed=21, max_tokens=32)):
        together = engine.generate(prompts, sp)
        alone = [engine.generate(p, sp) for p in prompts]
        for i, (a, b) in enumerate(zip(together, alone)):
            assert a.tokens == b.tokens, f"prompt {i}: the reply among eight differs from the reply alone"


# ---------------------------------------------------------------------------
# contexts of thousands of positions
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
def test_contexts_of_thousands_of_positions(dtype, tmp_path):
    """A GPT-2 with 4,100 positions (257 pages of 16 a request): block tables, context buckets,
    attention's splits and the prefill's walk over keys at four times GPT-2's own context. A
    request of 4,100 tokens and one of 2,500, most of each in one step and the last 32 one by
    one, in portions of up to 2,048 tokens, and mixed; every wanted row against the plain
    implementation. (That a far key is found among thousands, which random weights would
    average away, is the kernels' own test: test_attention_finds_one_far_key.)"""
    from liyab_amd.engine import EngineCore
    from liyab_amd.weights import write_random_model

    cfg = {"architectures": ["GPT2LMHeadModel"], "n_layer": 2, "n_embd": 64, "n_head": 2, "n_inner": 96, "vocab_size": 300,
           "n_positions": 4100, "layer_norm_epsilon": 1e-5, "activation_function": "gelu_new"}
    write_random_model(str(tmp_path), cfg, 31)
    config, tensors = plain.read_model(str(tmp_path))
    weights = tensors if dtype == "float32" else plain.round_weights_to_bf16(tensors)
    reqs = {"long": tt.random_tokens(1, 4100, 300), "mid": tt.random_tokens(2, 2500, 300)}
    refs = {rid: plain.forward(config, weights, t) for rid, t in reqs.items()}
    sparse = lambda steps: [dict(s, entries=[(r, t, w if len(t) < 64 else w[-3:]) for r, t, w in s["entries"]]) for s in steps]  # noqa: E731
    for label, steps in (("bulk+tail", tt.schedule_bulk_tail(reqs)), ("portions", sparse(tt.schedule_portions(reqs, (2048, 7, 1000, 2, 300)))),
                         ("mixed", sparse(tt.schedule_mixed(reqs, seed=4, decode_tail=6, portions=(700, 9, 1500, 64))))):
        core = EngineCore(str(tmp_path), dtype=dtype, page_size=16, max_tokens=tt.max_live_tokens(steps), max_requests=4)
        got = tt.run_schedule(core, steps)
        tt.check_against_plain(got, reqs, refs, TOL[dtype], f"4,100 positions {label} {dtype}", family="long context")
        core.manager.check()
        del core


@pytest.fixture(scope="module")
def positions_16640_model(tmp_path_factory):
    """A one-layer GPT-2 with 16,640 positions and its plain logits for one request that fills them
    and one short one (the plain attention takes a while at this length: made once)."""
    from liyab_amd.weights import write_random_model

    d = str(tmp_path_factory.mktemp("positions16640"))
    cfg = {"architectures": ["GPT2LMHeadModel"], "n_layer": 1, "n_embd": 32, "n_head": 2, "n_inner": 48, "vocab_size": 120,
           "n_positions": 16640, "layer_norm_epsilon": 1e-5, "activation_function": "gelu_new"}
    write_random_model(d, cfg, 77)
    config, tensors = plain.read_model(d)
    reqs = {"deep": tt.random_tokens(5, 16640, 120), "short": tt.random_tokens(6, 300, 120)}
    refs = {}
    for dtype in DTYPES:
        weights = tensors if dtype == "float32" else plain.round_weights_to_bf16(tensors)
        refs[dtype] = {rid: plain.forward(config, weights, t) for rid, t in reqs.items()}
    return d, reqs, refs


@pytest.mark.parametrize("mode,page_size", [("float32", 16), ("bfloat16", 16), ("bfloat16 batch-invariant", 16), ("float32", 8), ("bfloat16", 8)])
def test_contexts_past_16384_keys_and_tables_past_2048_pages(mode, page_size, positions_16640_model):
    """16,640 positions: past 16,384 keys the splits by position of the 32-bit path and of the
    batch-invariant mode are longer than 256 keys, so that sixteen of them still cover a request
    (a step of many tokens walks them in one workgroup, the last tokens are launched in splits);
    with pages of 8 a request's block table holds 2,080 pages, more than the fast attention
    kernels stage, and every step takes the plain kernel. A long request in portions of up to
    2,048 tokens with its last tokens one by one beside a short request's, against the plain
    implementation."""
    from liyab_amd.engine import EngineCore
    from liyab_amd.kernels import ops

    assert ops.invariant_chunk(16640) == 2048 and ops.invariant_chunk(1024) == 256 and ops.invariant_chunk(4097) == 512
    d, reqs, refs = positions_16640_model
    dtype = mode.split()[0]
    deep, short = reqs["deep"], reqs["short"]
    steps, at = [], 0
    for n in (2048, 2048, 1500, 2048, 2048, 2048, 2048, 2048, 700):  # 16,636; the last four one by one
        steps.append({"entries": [("deep", deep[at:at + n], [n - 2, n - 1])], "end": []})
        at += n
    steps.append({"entries": [("short", short[:296], [0, 295])], "end": []})
    for i in range(4):
        steps.append({"entries": [("deep", deep[at + i:at + i + 1], [0]), ("short", short[296 + i:297 + i], [0])],
                      "end": ["deep", "short"] if i == 3 else []})
    core = EngineCore(d, dtype=dtype, page_size=page_size, max_tokens=tt.max_live_tokens(steps), max_requests=2,
                      batch_invariant="invariant" in mode)
    assert core.manager.max_blocks == 16640 // page_size
    got = tt.run_schedule(core, steps)
    tt.check_against_plain(got, reqs, refs[dtype], TOL[dtype], f"16,640 positions, pages of {page_size}, {mode}", family="long context")
    core.manager.check()
    assert core.manager.pages_in_use() == 0


# ---------------------------------------------------------------------------
# layers far wider than GPT-2's own
# ---------------------------------------------------------------------------
@pytest.fixture(scope="module")
def width_4096_model(tmp_path_factory):
    """One model folder of width 4,096 for the tests below (writing it takes most of their time)."""
    from liyab_amd.weights import write_random_model

    d = str(tmp_path_factory.mktemp("width4096"))
    cfg = {"architectures": ["GPT2LMHeadModel"], "n_layer": 2, "n_embd": 4096, "n_head": 32, "n_inner": 16384, "vocab_size": 3000,
           "n_positions": 640, "layer_norm_epsilon": 1e-5, "activation_function": "gelu_new"}
    write_random_model(d, cfg, 5)
    return (d,) + tuple(plain.read_model(d))


@pytest.mark.parametrize("dtype", DTYPES)
def test_layers_of_width_4096(dtype, width_4096_model):
    """Width 4,096, 32 heads of 128, a feed-forward of 16,384: inner dimensions past what the
    kernel with the norm folded in takes (2,048), more output features than the streaming
    kernels take (8,192), heads of 128. Whole, most in one step with a tail token by token,
    and mixed, against the plain implementation."""
    from liyab_amd.engine import EngineCore

    d, config, tensors = width_4096_model
    weights = tensors if dtype == "float32" else plain.round_weights_to_bf16(tensors)
    reqs = {f"w{i}": tt.random_tokens(40 + i, n, 3000) for i, n in enumerate([200, 37, 3, 90])}
    refs = {rid: plain.forward(config, weights, t) for rid, t in reqs.items()}
    for label, steps in (("whole", tt.schedule_whole(reqs)), ("mixed", tt.schedule_mixed(reqs, seed=3, decode_tail=6)),
                         ("bulk+tail", tt.schedule_bulk_tail(reqs, tail=8))):
        core = EngineCore(d, dtype=dtype, page_size=16, max_tokens=tt.max_live_tokens(steps), max_requests=4)
        got = tt.run_schedule(core, steps)
        tt.check_against_plain(got, reqs, refs, TOL[dtype], f"width 4,096 {label} {dtype}", family="sizes:wide")
        core.manager.check()
        del core


def test_few_heads_over_many_keys_finish_their_own_splits(width_4096_model):
    """One request of 600 positions at 32 heads of 128, its tail token by token: the projection
    of this width is not cut over its inner dimension, so nobody merges attention's splits for
    it, and with 32 (token, head) pairs the step cuts the keys into 8 splits and merges them
    itself (ops.decode_plan)."""
    from liyab_amd.engine import EngineCore
    from liyab_amd.kernels import ops

    d, config, tensors = width_4096_model
    assert ops.decode_plan(1, 32, 1024) == (8, 4) and ops.k_parts(1, 4096, 4096) == 1
    weights = plain.round_weights_to_bf16(tensors)
    reqs = {"deep": tt.random_tokens(77, 600, 3000)}
    refs = {rid: plain.forward(config, weights, t) for rid, t in reqs.items()}
    steps = tt.schedule_bulk_tail(reqs, tail=12)
    core = EngineCore(d, dtype="bfloat16", page_size=16, max_tokens=tt.max_live_tokens(steps), max_requests=2)
    got = tt.run_schedule(core, steps)
    tt.check_against_plain(got, reqs, refs, TOL["bfloat16"], "width 4,096, 600 positions, tail token by token", family="sizes:wide")
    core.manager.check()
