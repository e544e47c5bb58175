"""Decode and prefill throughput of the engine on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 8] [--size small|medium|xl] [--layers L]
    python bench.py --sequences 1,2,4,8 [-n 128]     # together against in turns, and whether replies are the same
    python bench.py --prefill-tokens 512,2048,8192   # prefill tokens a second per length

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
WEIGHT_SEEDS = {"small": 10, "medium": 20, "xl": 30}
SIZES = {"small": {}, "medium": {"n_layer": 24, "n_embd": 1024, "n_head": 16, "n_inner": 4096},
         "xl": {"n_layer": 48, "n_embd": 1600, "n_head": 25, "n_inner": 6400}}


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


def make_engine(model_dir, dtype, batch, ctx):
    from liyab_amd import Engine

    pages = batch * (-(-ctx // 64)) + 4
    return Engine(model_dir, dtype=dtype, page_size=64, num_pages=pages, max_num_seqs=max(batch, 2),
                  max_batched_tokens=max(2048, batch), prefill_chunk=1024, ctx=ctx)


def decode_run(engine, cfg, batch, prompt_len, steps, warmup, seed=11):
    """(tokens/s, ms/step, bytes/step) over `steps` decode steps of `batch` requests."""
    import numpy as np
    import torch

    from liyab_amd import SamplingParams

    rng = np.random.default_rng(seed)
    engine.stop_at_eos = False
    for i in range(batch):
        prompt = rng.integers(0, cfg["vocab_size"], prompt_len).tolist()
        engine.add_request(prompt, SamplingParams(temperature=0.0, max_tokens=steps + warmup + 1), rid=f"b{batch}-{i}")
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
    bytes_per_step = weight_bytes(cfg, elt) + kv_positions * kv_bytes_per_position(cfg, elt) / steps
    for r in list(engine.scheduler.running):
        engine.abort(r.rid)
    return batch * steps / dt, dt * 1e3 / steps, bytes_per_step


def prefill_run(engine, cfg, prompt_lens, repeat=5, seed=12):
    """Best of `repeat`: (tokens/s, ms) of one step that holds the whole prompts."""
    import numpy as np
    import torch

    from liyab_amd.engine import StepItem

    rng = np.random.default_rng(seed)
    prompts = [rng.integers(0, cfg["vocab_size"], n).tolist() for n in prompt_lens]
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
    ap.add_argument("--size", default="small", choices=sorted(SIZES), help="GPT-2 small's sizes (the default), medium's or XL's")
    ap.add_argument("--layers", type=int, default=0, help="fewer layers than the configuration has, if needed")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--prompt", type=int, default=512)
    ap.add_argument("--no-points", action="store_true", help="skip the batch 1 / 64 points and the prefill")
    ap.add_argument("--prefill-only", action="store_true", help="run only the prefill of 2,048 tokens (for profiling)")
    ap.add_argument("--prefill-tokens", default="", help="e.g. 512,2048,8192: best-of-5 prefill tokens a second per length, "
                    "in prompts of up to 1,024 tokens (the reference's liyab-bench --prefill --tokens)")
    ap.add_argument("--sequences", default="", help="e.g. 1,2,4: that many sequences together against one after the other "
                    "(the reference's liyab-seq-bench): tokens a second both ways and whether every reply equals its reply alone")
    ap.add_argument("-n", type=int, default=128, help="tokens generated per sequence with --sequences")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported")
        return 2
    import torch

    from liyab_amd.weights import write_random_model

    cfg = dict(SMALL, **SIZES[args.size])
    full_layers = cfg["n_layer"]
    if args.layers:
        cfg["n_layer"] = args.layers
    ctx = cfg["n_positions"]
    steps = max(1, min(args.steps, ctx - args.prompt - args.warmup))
    short = "bf16" if args.dtype == "bfloat16" else "fp32"
    with tempfile.TemporaryDirectory() as d:
        write_random_model(d, cfg, WEIGHT_SEEDS[args.size], dtype="bfloat16" if short == "bf16" else "float32")
        slots = max(args.batch, 64 if not args.no_points else args.batch)
        if args.prefill_tokens:
            slots = max(slots, max(-(-int(x) // ctx) for x in args.prefill_tokens.split(",")))
        engine = make_engine(d, args.dtype, slots, ctx)
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
                       "global_batch": args.batch, "seq_len": ctx, "prompt_len": args.prompt, "page_size": 64,
                       "weights_seed": WEIGHT_SEEDS[args.size], "ids_seed": 11, "parallelism": "single-gpu"},
            "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                         "frac": round(achieved / HBM_PEAK_GBS, 4)},
        }
        if not args.no_points:
            lens = [1024, 1024]
            ptps, pms = prefill_run(engine, cfg, lens)
            flops = prefill_flops(cfg, lens, len(lens))
            out["prefill"] = {"value": round(ptps, 1), "tokens": sum(lens), "ms": round(pms, 4),
                              "frac": round(flops / (pms * 1e-3) / MFMA_PEAK[short], 4)}
            points = {}
            for b in (1, 64):
                k = min(steps, 256)
                t, _, _ = decode_run(engine, cfg, b, args.prompt, k, args.warmup)
                points[f"decode_b{b}"] = round(t, 1)
            out["points"] = points
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
