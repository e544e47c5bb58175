"""Decode and prefill throughput of the engine on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 8] [--size small|medium|large|xl|wide] [--layers L]
    python bench.py --sequences 1,2,4,8 [-n 128]     # together against in turns, and whether replies are the same
    python bench.py --prefill-tokens 512,2048,8192   # prefill tokens a second per length
    python bench.py --workload medium16|xl64         # the continuous-batching and the batch-64 workloads of the larger sizes
    python bench.py --link-floor                     # what one dependent kernel of a replayed graph costs at least
    python bench.py --product 4096,4096,16384,8,15   # one product in tiles of 128 x 128 and of 256 x 256

The default run has GPT-2 small's layer sizes (12 layers, width 768, 12 heads
of 64, feed-forward 3072, vocabulary 50257, 1024 positions) with random
weights in bfloat16, a batch of 8 requests with 512-token prompts decoding
towards 1,024 tokens. A step is one decode step of the whole engine loop:
scheduler, model step, sampling, tokens back on the host. It prints one JSON
line: decoded tokens a second, the prefill of 2,048 tokens (two prompts of
1,024), the decode step's share of the HBM roofline (bytes it has to read:
every weight once and the live requests' cache, over its time), and decoding
at batch 1 and 64. Token ids are seeded synthetic ones; no dataset is used.
The reference measures the same way: tokens a second beside a ceiling from
the bytes a decoded token must read (src/core/model_bytes.h:1-5,
docs/guide/development.md:115-122) and prefill over synthetic ids
(tools/liyab_bench.cpp:87-169).
"""

import argparse
import json
import os
import sys
import tempfile
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X, published
MFMA_PEAK = {"bf16": 2.5e15, "fp32": 157.3e12}

SMALL = {"architectures": ["GPT2LMHeadModel"], "model_type": "gpt2", "n_layer": 12, "n_embd": 768, "n_head": 12,
         "n_inner": 3072, "vocab_size": 50257, "n_positions": 1024, "layer_norm_epsilon": 1e-5,
         "activation_function": "gelu_new", "tie_word_embeddings": True}
# GPT-2's other sizes, for --size: the layer sizes and, with them, the number of layers
# ("wide": no GPT-2 of anybody's, but the architecture at layer sizes where a decode step is bound by the weights' bytes, not by
# its chain of kernels: 403 MB of matrices a layer; run it with --layers 8 or so)
WEIGHT_SEEDS = {"small": 10, "medium": 20, "large": 25, "xl": 30, "wide": 40}
SIZES = {"small": {}, "medium": {"n_layer": 24, "n_embd": 1024, "n_head": 16, "n_inner": 4096},
         "large": {"n_layer": 36, "n_embd": 1280, "n_head": 20, "n_inner": 5120},
         "xl": {"n_layer": 48, "n_embd": 1600, "n_head": 25, "n_inner": 6400},
         "wide": {"n_layer": 32, "n_embd": 4096, "n_head": 32, "n_inner": 16384}}


def weight_bytes(cfg, elt):
    d, F, V, L = cfg["n_embd"], cfg["n_inner"], cfg["vocab_size"], cfg["n_layer"]
    matrices = L * (3 * d * d + d * d + 2 * d * F) + V * d  # the tied table is read once, as the head
    vectors = L * (3 * d + d + F + d + 4 * d) + 2 * d  # biases and norm vectors, float32
    return matrices * elt + vectors * 4


def kv_bytes_per_position(cfg, elt):
    return 2 * cfg["n_layer"] * cfg["n_embd"] * elt


def prefill_flops(cfg, prompt_lens, logit_rows):
    d, F, V, L = cfg["n_embd"], cfg["n_inner"], cfg["vocab_size"], cfg["n_layer"]
    n = sum(prompt_lens)
    flops = 2.0 * n * L * (3 * d * d + d * d + 2 * d * F)
    for t in prompt_lens:
        flops += L * 2.0 * d * t * (t + 1)  # q.k and p.v over the causal half
    return flops + 2.0 * logit_rows * d * V


def make_engine(model_dir, dtype, batch, ctx, page_size=64, prefill_chunk=1024, batch_invariant=False, phases=False):
    from liyab_amd import Engine

    pages = batch * (-(-ctx // page_size)) + 4
    return Engine(model_dir, dtype=dtype, page_size=page_size, num_pages=pages, max_num_seqs=max(batch, 2),
                  max_batched_tokens=max(2048, batch), prefill_chunk=prefill_chunk, ctx=ctx, batch_invariant=batch_invariant,
                  phases=phases)


def decode_run(engine, cfg, batch, prompt_len, steps, warmup, seed=11):
    """(tokens/s, ms/step, bytes/step) over `steps` decode steps of `batch` requests."""
    import numpy as np
    import torch

    from liyab_amd import SamplingParams

    rng = np.random.default_rng(seed)
    engine.stop_at_eos = False
    for i in range(batch):
        prompt = rng.integers(0, cfg["vocab_size"], prompt_len).tolist()
        # (requests that go on for some steps past the timed ones: a request about to reach its last
        # token is waited for, not run ahead of, and that wait is no part of a decode step)
        engine.add_request(prompt, SamplingParams(temperature=0.0, max_tokens=steps + warmup + 8), rid=f"b{batch}-{i}")
    while any(r.remaining > 1 or not r.generated for r in engine.scheduler.running) or engine.scheduler.waiting:
        engine.step()  # prompts, until every request is decoding
    for _ in range(warmup):
        engine.step()
    contexts = [r.computed for r in engine.scheduler.running]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        engine.step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    elt = 2 if engine.core.dtype == torch.bfloat16 else 4
    # each timed step s reads the cache of positions [0, context + s] of every request
    kv_positions = sum(c * steps + steps * (steps + 1) // 2 for c in contexts)
    bytes_per_step = weight_bytes(cfg, elt) + kv_positions * kv_bytes_per_position(cfg, elt) / max(steps, 1)
    for r in list(engine.scheduler.running):
        engine.abort(r.rid)
    return batch * steps / dt, dt * 1e3 / max(steps, 1), bytes_per_step


def workload_run(engine, cfg, prompts, params_of, label):
    """A whole workload through the engine's loop: requests arrive together, prompts go in portions
    beside decoding requests. Returns generated tokens a second, all tokens (prompt and generated)
    a second, and the share of the HBM roofline: the bytes every step has to read (each weight
    once, and the cache of the positions its requests hold) over the whole time."""
    import torch

    elt = 2 if engine.core.dtype == torch.bfloat16 else 4
    w_bytes, kv_pos = weight_bytes(cfg, elt), kv_bytes_per_position(cfg, elt)
    engine.stop_at_eos = False
    rids = [engine.add_request(p, params_of(i), rid=f"{label}-{i}") for i, p in enumerate(prompts)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    steps = bytes_read = 0
    while engine.has_unfinished():
        before = engine.core.step_fn.steps
        engine.step()
        if engine.core.step_fn.steps > before:
            h = engine.core.step_fn.last_context.host
            bytes_read += w_bytes + kv_pos * sum(f + q for f, q in zip(h.first_pos, h.q_lens))
            steps += 1
    engine.flush()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    results = [engine.result(r) for r in rids]
    for r in rids:
        engine.release(r)
    generated = sum(len(r.tokens) for r in results)
    prompt_tokens = sum(len(p) for p in prompts)
    return {"generated_tok_s": round(generated / dt, 1), "all_tok_s": round((generated + prompt_tokens) / dt, 1),
            "seconds": round(dt, 4), "steps": steps, "ms_per_step": round(dt * 1e3 / max(steps, 1), 4),
            "generated": generated, "prompt_tokens": prompt_tokens,
            "preemptions": sum(r.stats.preemptions for r in results),
            "roofline_frac": round(bytes_read / dt / 1e9 / HBM_PEAK_GBS, 4)}, [r.tokens for r in results]


def product_run(M, N, K, tiles, device="cuda:0", reps=30):
    """One product a[M, K] . w[N, K]^T + bias in bfloat16 (outputs bfloat16), as the tiled matrix-core
    kernel runs it in the tiles named (0: the kernel's own choice; 2 and 6: 64 x 64, 8: 128 x 128,
    15: 256 x 256): microseconds and TFLOP/s each."""
    import torch

    from liyab_amd.kernels import ops

    dev = torch.device(device)
    a = torch.randn(M, K, device=dev).bfloat16()
    w = (torch.randn(N, K, device=dev) * 0.02).bfloat16()
    bias = torch.randn(N, device=dev)
    out = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
    runs = []
    for tile in tiles:
        for _ in range(3):
            ops.gemm_mfma_dl(a, w, bias, out=out, tile=tile)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            ops.gemm_mfma_dl(a, w, bias, out=out, tile=tile)
        e1.record()
        torch.cuda.synchronize()
        us = e0.elapsed_time(e1) / reps * 1e3
        runs.append({"tile": tile, "us": round(us, 1), "tflops": round(2.0 * M * N * K / us / 1e6, 1)})
    return {"metric": "one product, bfloat16", "M": M, "N": N, "K": K, "runs": runs}


def link_floor(device="cuda:0", links=100):
    """What a dependent kernel costs at least inside a replayed graph, measured with the library's
    own kernels: a chain of kernels that each write one word (the distance from one kernel's end
    to the next one's start), and a chain of norms over 8 rows of 768 in which each reads what the
    one before wrote (a boundary, a first read of fresh data, a few hundred cycles of work, a write)."""
    import torch

    from liyab_amd.kernels import ops

    dev = torch.device(device)
    one = torch.zeros(64, dtype=torch.int32, device=dev)
    a = torch.randn(8, 768, device=dev)
    b = torch.empty_like(a)
    w, bias = torch.ones(768, device=dev), torch.zeros(768, device=dev)
    out = {}
    for name, body in (("a kernel that writes one word", lambda i: ops.fill_(one[:1], i)),
                       ("a norm of 8 rows of 768 that reads the one before", lambda i: ops.layernorm(b if i % 2 == 0 else a, a if i % 2 == 0 else b, w, bias, 1e-5))):
        for i in range(3):
            body(i)
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            for i in range(links):
                body(i)
        best = float("inf")
        for _ in range(6):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            g.replay()
            e1.record()
            e1.synchronize()
            best = min(best, e0.elapsed_time(e1))
        out[name] = round(best * 1e3 / links, 3)
    return {"metric": "microseconds a dependent kernel of a replayed graph", "links": links, "us_per_link": out}


def copy_bandwidth(device="cuda:0", mbytes=1024, repeat=5):
    """GB/s of a device-to-device copy of `mbytes` (bytes read plus bytes written over the best
    time): what this machine's memory gives a plain stream, beside the published peak that the
    roofline shares are taken against (the reference measures its read ceiling the same way,
    tools/liyab_bench.cpp:1-9)."""
    import torch

    n = mbytes * (1 << 20) // 4
    a = torch.empty(n, dtype=torch.float32, device=device).normal_()
    b = torch.empty_like(a)
    best = float("inf")
    for _ in range(repeat + 1):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        b.copy_(a)
        e1.record()
        e1.synchronize()
        best = min(best, e0.elapsed_time(e1))
    return 2.0 * n * 4 / (best * 1e-3) / 1e9


def prefill_run(engine, cfg, prompt_lens, repeat=5, seed=12):
    """Best of `repeat`: (tokens/s, ms) of one step that holds the whole prompts."""
    import numpy as np
    import torch

    from liyab_amd.engine import StepItem

    rng = np.random.default_rng(seed)
    prompts = [rng.integers(0, cfg["vocab_size"], n) for n in prompt_lens]  # arrays of ids, as the scheduler hands portions over
    best = float("inf")
    for it in range(repeat + 2):
        for i in range(len(prompts)):
            engine.core.open(f"p{i}")
        items = [StepItem(f"p{i}", p, [len(p) - 1]) for i, p in enumerate(prompts)]
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        engine.core.step(items)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        for i in range(len(prompts)):
            engine.core.close(f"p{i}")
        if it >= 2:
            best = min(best, dt)
    n = sum(prompt_lens)
    return n / best, best * 1e3


def ttft_run(engine, cfg, prompt_len=512, repeat=6, seed=14):
    """An idle engine and one prompt: milliseconds until step() has launched everything (the host's
    share), the step's kernels on the device (events around it), and until the first token is on the
    host; best of `repeat`, prompts of prompt_len - 0, 1, 2, ... tokens. First with everything the
    engine knows of earlier steps forgotten before each prompt, so that its step is launched kernel by
    kernel (`first_sight_*`: a size the engine has not seen); then as they come: the prompts' steps are
    padded to one size, captured after three sights and replayed (`ms`, `host_ms`, `device_ms`)."""
    import numpy as np
    import torch

    from liyab_amd import SamplingParams

    rng = np.random.default_rng(seed)
    engine.stop_at_eos = False

    def one(length):
        prompt = rng.integers(0, cfg["vocab_size"], length).tolist()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        rid = engine.add_request(prompt, SamplingParams(temperature=0.0, max_tokens=1))
        e0.record()
        engine.step()
        e1.record()
        t1 = time.perf_counter()
        while engine.has_unfinished():
            engine.step()
        engine.flush()
        t2 = time.perf_counter()
        torch.cuda.synchronize()
        engine.release(rid)
        return (t1 - t0) * 1e3, e0.elapsed_time(e1), (t2 - t0) * 1e3

    out = {"prompt_len": prompt_len}
    for label, forget in (("first_sight_", True), ("", False)):
        best = [float("inf")] * 3
        for it in range(repeat + 4):
            if forget:
                engine.core.step_fn.forget_graphs()
            got = one(prompt_len - it % 8)
            if it >= 4:
                best = [min(a, b) for a, b in zip(best, got)]
        out.update({label + "host_ms": round(best[0], 4), label + "device_ms": round(best[1], 4), label + "ms": round(best[2], 4)})
    return out


def sequences_run(engine, cfg, counts, prompt_len, n_new, seed=13):
    """Several sequences generated together against the same sequences one after the other, as
    the reference's liyab-seq-bench reports them (tools/liyab_seq_bench.cpp:1-32): total tokens
    a second both ways, the gain, and whether every reply equals its reply alone. Greedy, and
    with a seeded temperature."""
    import numpy as np
    import torch

    from liyab_amd import SamplingParams

    rng = np.random.default_rng(seed)
    engine.stop_at_eos = False
    out = []
    for count in counts:
        prompts = [rng.integers(0, cfg["vocab_size"], prompt_len).tolist() for _ in range(count)]
        for name, make in (("greedy", lambda i: SamplingParams(temperature=0.0, max_tokens=n_new)),
                           ("temperature 0.8", lambda i: SamplingParams(temperature=0.8, top_k=40, top_p=0.95, seed=100 + i, max_tokens=n_new))):
            for _ in range(2):  # the second run replays captured graphs
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                together = engine.generate(prompts, [make(i) for i in range(count)])
                torch.cuda.synchronize()
                t_together = time.perf_counter() - t0
                t0 = time.perf_counter()
                alone = [engine.generate([p], [make(i)])[0] for i, p in enumerate(prompts)]
                torch.cuda.synchronize()
                t_turns = time.perf_counter() - t0
            total = sum(len(r.tokens) for r in together)
            out.append({"sequences": count, "sampling": name, "together_tok_s": round(total / t_together, 1),
                        "in_turns_tok_s": round(total / t_turns, 1), "gain": round(t_turns / t_together, 2),
                        "same": all(a.tokens == b.tokens for a, b in zip(together, alone))})
    return {"metric": "sequences together against in turns", "prompt_len": prompt_len, "new_tokens": n_new, "runs": out}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=504)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--size", default="small", choices=sorted(SIZES), help="GPT-2 small's sizes (the default), medium's, large's or XL's; or layers of width 4,096")
    ap.add_argument("--layers", type=int, default=0, help="fewer layers than the configuration has, if needed")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--prompt", type=int, default=512)
    ap.add_argument("--positions", type=int, default=0, help="a longer context than the size's own (the position table grows), e.g. 8192 with --prompt 7000")
    ap.add_argument("--no-points", action="store_true", help="skip the batch 1 / 64 points and the prefill")
    ap.add_argument("--prefill-only", action="store_true", help="run only the prefill of 2,048 tokens (for profiling)")
    ap.add_argument("--prefill-tokens", default="", help="e.g. 512,2048,8192: best-of-5 prefill tokens a second per length, "
                    "in prompts of up to 1,024 tokens (the reference's liyab-bench --prefill --tokens)")
    ap.add_argument("--sequences", default="", help="e.g. 1,2,4: that many sequences together against one after the other "
                    "(the reference's liyab-seq-bench): tokens a second both ways and whether every reply equals its reply alone")
    ap.add_argument("-n", type=int, default=128, help="tokens generated per sequence with --sequences")
    ap.add_argument("--workload", default="", choices=["", "medium16", "xl64"],
                    help="medium16: GPT-2 medium's sizes, 16 requests with prompts of 64 to 1,023 tokens, portions of 256, 128 greedy "
                         "tokens each; xl64: GPT-2 XL's sizes, 64 requests with prompts of 256 tokens decoding to 1,024, greedy and at temperature 1")
    ap.add_argument("--page-size", type=int, default=64, help="positions a cache page (default 64; the engine's own default is 16)")
    ap.add_argument("--batch-invariant", action="store_true", help="kernels chosen from sizes and positions only (reproducible bfloat16 replies)")
    ap.add_argument("--product", default="", help="M,N,K[,tile,...]: time one bfloat16 product in the tiled kernel's tiles (0: its own choice, 6: 64 x 64, 8: 128 x 128, 15: 256 x 256)")
    ap.add_argument("--link-floor", action="store_true", help="measure what one dependent kernel of a replayed graph costs at least")
    ap.add_argument("--phases", action="store_true", help="device milliseconds per phase of the forward pass (embed, attention, dense_ffn, lm_head) a decode step "
                    "and a prefill of 2,048 tokens, as the reference's command line prints them (tools/liyab_cli.cpp:198-211); steps run kernel by kernel, without graphs")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported")
        return 2
    import torch

    from liyab_amd.weights import write_random_model

    if args.product:
        sizes = [int(x) for x in args.product.split(",")]
        print(json.dumps(product_run(sizes[0], sizes[1], sizes[2], sizes[3:] or [0])))
        return 0
    if args.link_floor:
        print(json.dumps(link_floor()))
        return 0
    if args.workload:
        args.size = "medium" if args.workload == "medium16" else "xl"
    cfg = dict(SMALL, **SIZES[args.size])
    full_layers = cfg["n_layer"]
    if args.layers:
        cfg["n_layer"] = args.layers
    if args.positions:
        cfg["n_positions"] = args.positions
    ctx = cfg["n_positions"]
    steps = max(1, min(args.steps, ctx - args.prompt - args.warmup))
    short = "bf16" if args.dtype == "bfloat16" else "fp32"
    with tempfile.TemporaryDirectory() as d:
        write_random_model(d, cfg, WEIGHT_SEEDS[args.size], dtype="bfloat16" if short == "bf16" else "float32")
        slots = max(args.batch, 64 if not args.no_points else args.batch)
        if args.prefill_tokens:
            slots = max(slots, max(-(-int(x) // ctx) for x in args.prefill_tokens.split(",")))
        if args.workload:
            import numpy as np

            from liyab_amd import SamplingParams

            layers_note = {"n_layer": cfg["n_layer"], "n_layer_full": full_layers}
            if args.workload == "medium16":
                # the continuous-batching workload at GPT-2 medium's sizes: 16 requests, prompt lengths uniform in [64, 1024) and ids
                # from seed 21, continuously batched with portions of 256, 128 greedy tokens each (capped at the positions)
                rng = np.random.default_rng(21)
                lens = rng.integers(64, 1024, 16).tolist()
                prompts = [rng.integers(0, cfg["vocab_size"], n).tolist() for n in lens]
                engine = make_engine(d, args.dtype, 16, ctx, page_size=args.page_size, prefill_chunk=256, batch_invariant=args.batch_invariant)
                engine.warmup()
                runs = {}
                for rep in range(2):  # the second run finds its recurring shapes captured
                    runs["greedy"], _ = workload_run(engine, cfg, prompts, lambda i: SamplingParams(temperature=0.0, max_tokens=128), f"m{rep}")
                print(json.dumps({"metric": "GPT-2 medium sizes: 16 requests, prompts of 64 to 1,023 tokens in portions of 256, 128 greedy tokens each",
                                  "dtype": short, "data": "synthetic", "page_size": args.page_size, **layers_note,
                                  "prompt_lens": lens, "runs": runs}))
            else:
                # the batch-64 workload at GPT-2 XL's sizes: 64 requests, prompts of 256 ids from seed 31, decoding to 1,024
                # positions, greedy and at temperature 1
                rng = np.random.default_rng(31)
                prompts = [rng.integers(0, cfg["vocab_size"], 256).tolist() for _ in range(64)]
                engine = make_engine(d, args.dtype, 64, ctx, page_size=args.page_size, prefill_chunk=256, batch_invariant=args.batch_invariant)
                engine.warmup()
                runs = {}
                n_new = ctx - 256 + 1
                for name, make in (("greedy", lambda i: SamplingParams(temperature=0.0, max_tokens=n_new)),
                                   ("temperature 1.0", lambda i: SamplingParams(temperature=1.0, top_k=0, top_p=1.0, seed=1000 + i, max_tokens=n_new))):
                    runs[name], _ = workload_run(engine, cfg, prompts, make, name[:1])
                print(json.dumps({"metric": "GPT-2 XL sizes: 64 requests, prompts of 256 tokens decoding to 1,024 positions",
                                  "dtype": short, "data": "synthetic", "page_size": args.page_size, **layers_note, "runs": runs}))
            return 0
        engine = make_engine(d, args.dtype, slots, ctx, page_size=args.page_size, batch_invariant=args.batch_invariant)
        if args.prefill_tokens:
            runs = []
            for total in [int(x) for x in args.prefill_tokens.split(",")]:
                lens = [ctx] * (total // ctx) + ([total % ctx] if total % ctx else [])
                ptps, pms = prefill_run(engine, cfg, lens)
                flops = prefill_flops(cfg, lens, len(lens))
                runs.append({"tokens": total, "prompts": len(lens), "value": round(ptps, 1), "ms": round(pms, 4),
                             "frac": round(flops / (pms * 1e-3) / MFMA_PEAK[short], 4)})
            print(json.dumps({"metric": f"prefill tok/s (GPT-2 {args.size} sizes)", "dtype": short, "runs": runs}))
            return 0
        if args.sequences:
            print(json.dumps(sequences_run(engine, cfg, [int(x) for x in args.sequences.split(",")], args.prompt, args.n)))
            return 0
        if args.phases:
            timed = make_engine(d, args.dtype, max(args.batch, 2), ctx, page_size=args.page_size, batch_invariant=args.batch_invariant, phases=True)
            k = min(steps, 64)
            decode_run(timed, cfg, args.batch, args.prompt, 4, 2)  # every kernel has run once
            timed.phases_ms(reset=True)
            tps, ms, _ = decode_run(timed, cfg, args.batch, args.prompt, k, 0, seed=12)
            whole = timed.phases_ms(reset=True)  # the prompts of the run, too: taken off below
            prefill_run(timed, cfg, [1024, 1024], repeat=1)
            prefill = timed.phases_ms(reset=True)
            per = lambda table, n: {name: round(v / n, 4) for name, v in table.items()}  # noqa: E731
            # the prompts of the decode run went through the same timer: one step of `batch` prompts of args.prompt tokens
            timed.phases_ms(reset=True)
            decode_run(timed, cfg, args.batch, args.prompt, 0, 0, seed=12)
            prompts_only = timed.phases_ms(reset=True)
            decode = {name: max(whole.get(name, 0.0) - prompts_only.get(name, 0.0), 0.0) for name in whole}
            print(json.dumps({"metric": f"device ms per phase (GPT-2 {args.size} sizes, {short}; steps launched kernel by kernel)",
                              "decode_step": {"batch": args.batch, "steps": k, "phases_ms": per(decode, k), "ms_per_step_wall": round(ms, 4)},
                              "prefill_2048": {"phases_ms": per(prefill, 3)}}))
            return 0
        if args.prefill_only:
            ptps, pms = prefill_run(engine, cfg, [1024, 1024], repeat=20)
            print(json.dumps({"prefill": {"value": round(ptps, 1), "tokens": 2048, "ms": round(pms, 4)}}))
            return 0
        tps, ms, bytes_per_step = decode_run(engine, cfg, args.batch, args.prompt, steps, args.warmup)
        achieved = bytes_per_step / (ms * 1e-3) / 1e9
        out = {
            "metric": f"decode tok/s (GPT-2 {args.size} sizes, batch {args.batch}, {args.prompt}-token prompts decoding to {ctx})",
            "value": round(tps, 1), "unit": "tok/s", "n_gpus": 1, "steps": steps, "warmup": args.warmup,
            "ms_per_step": round(ms, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
            "dtype": short, "data": "synthetic",
            "config": {"model": f"gpt2-{args.size}-sizes-random-weights", "n_layer": cfg["n_layer"], "n_layer_full": full_layers,
                       "n_embd": cfg["n_embd"], "n_head": cfg["n_head"], "head_dim": cfg["n_embd"] // cfg["n_head"],
                       "n_inner": cfg["n_inner"], "vocab_size": cfg["vocab_size"], "n_positions": cfg["n_positions"],
                       "global_batch": args.batch, "seq_len": ctx, "prompt_len": args.prompt, "page_size": args.page_size,
                       "batch_invariant": bool(args.batch_invariant),
                       "weights_seed": WEIGHT_SEEDS[args.size], "ids_seed": 11, "parallelism": "single-gpu"},
            "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                         "frac": round(achieved / HBM_PEAK_GBS, 4)},
        }
        if not args.no_points:
            out["roofline"]["measured_copy"] = round(copy_bandwidth(), 1)  # a 1 GiB device-to-device copy on this machine, GB/s
        if not args.no_points:
            lens = [1024, 1024]
            ptps, pms = prefill_run(engine, cfg, lens)
            flops = prefill_flops(cfg, lens, len(lens))
            out["prefill"] = {"value": round(ptps, 1), "tokens": sum(lens), "ms": round(pms, 4),
                              "frac": round(flops / (pms * 1e-3) / MFMA_PEAK[short], 4)}
            out["ttft"] = ttft_run(engine, cfg, min(args.prompt, ctx - 16))
            # every point over at least 64 steps after at least 3 of its own shape, whatever --steps says: fewer do
            # not outlast the first sight of a shape (an eager run, then a capture)
            points = {}
            k, w = min(max(steps, 64), 256, ctx - args.prompt - 8), max(args.warmup, 3)
            for b in (1, 64):
                t, pms_b, pbytes = decode_run(engine, cfg, b, args.prompt, k, w)
                points[f"decode_b{b}"] = round(t, 1)
                points[f"decode_b{b}_ms_per_step"] = round(pms_b, 4)
                points[f"decode_b{b}_mbytes_per_step"] = round(pbytes / 1e6, 1)
                points[f"decode_b{b}_roofline_frac"] = round(pbytes / (pms_b * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)
            points["steps_per_point"] = k
            if args.page_size != 16:
                # the headline batch again with pages of 16 positions, the engine's own default
                small_pages = make_engine(d, args.dtype, args.batch, ctx, page_size=16, batch_invariant=args.batch_invariant)
                t, pms_b, _ = decode_run(small_pages, cfg, args.batch, args.prompt, k, w)
                points[f"decode_b{args.batch}_page16"] = round(t, 1)
                points[f"decode_b{args.batch}_page16_ms_per_step"] = round(pms_b, 4)
                del small_pages
            # the headline batch in the engine's two other modes: replies that do not depend on the batch, and the 32-bit path
            others = []
            if not args.batch_invariant and short == "bf16":
                others.append((f"decode_b{args.batch}_batch_invariant", args.dtype, True))
            if short == "bf16":
                others.append((f"decode_b{args.batch}_fp32", "float32", False))
            del engine
            for name, dtype, invariant in others:
                other = make_engine(d, dtype, args.batch, ctx, page_size=args.page_size, batch_invariant=invariant)
                t, pms_b, _ = decode_run(other, cfg, args.batch, args.prompt, k, w)
                points[name] = round(t, 1)
                points[name + "_ms_per_step"] = round(pms_b, 4)
                del other
            out["points"] = points
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
