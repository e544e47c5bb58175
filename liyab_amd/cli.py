"""Command line, in the manner of the reference's liyab-cli.

Option names and meanings follow `tools/liyab_cli.cpp:242-335` where the
reference has them: -m, -p, -n (default 128), --temp (0.8, 0 = greedy),
--top-k (40), --top-p (0.95), --seed (random), --ctx, --json, --tokenize.
The reference's --kv picks the cache's row type; here --dtype picks the
precision of the whole path. The engine works on token ids, so -p takes
ids ("5,17,3" or "5 17 3"); --prompt-ids and --prompt-file are synonyms.
The summary on stderr and the --json line carry the reference's fields
(`tools/liyab_cli.cpp:145-162, 218-240`).
"""

from __future__ import annotations

import argparse
import json
import re
import sys
import tempfile
import time


def _ids(text: str):
    parts = [p for p in re.split(r"[\s,]+", text.strip()) if p]
    try:
        return [int(p) for p in parts]
    except ValueError:
        raise SystemExit("liyab-cli: the prompt must be token ids (this engine has no tokenizer): e.g. -p 5,17,3")


def build_parser() -> argparse.ArgumentParser:
    ap = argparse.ArgumentParser(prog="liyab-cli", description="Generate tokens with a model folder (config.json + model.safetensors) on one MI355X.")
    ap.add_argument("-m", "--model", help="model folder (config.json + model.safetensors)")
    ap.add_argument("-p", "--prompt", "--prompt-ids", dest="prompt", help="prompt as token ids, e.g. 5,17,3")
    ap.add_argument("--prompt-file", help="file holding the prompt's token ids")
    ap.add_argument("-n", type=int, default=128, dest="n", help="max new tokens (default 128)")
    ap.add_argument("--temp", type=float, default=0.8, help="temperature, 0 = greedy (default 0.8)")
    ap.add_argument("--top-k", type=int, default=40, help="(default 40)")
    ap.add_argument("--top-p", type=float, default=0.95, help="(default 0.95)")
    ap.add_argument("--seed", type=int, default=0, help="RNG seed (default random)")
    ap.add_argument("--ctx", type=int, default=None, help="context length (default: the model's)")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32", "bf16", "fp32"],
                    help="precision of the whole path (default bfloat16)")
    ap.add_argument("--json", action="store_true", help="stdout: one JSON line after loading and one for the generation")
    ap.add_argument("--tokenize", action="store_true", help="print the prompt's token ids and exit")
    ap.add_argument("--phases", action="store_true",
                    help="time the device per phase of the forward pass (phases_ms in --json, ms per token on stderr); slower: no graphs")
    ap.add_argument("--device", default="cuda:0")
    ap.add_argument("--page-size", type=int, default=16, help="tokens per cache page (default 16)")
    ap.add_argument("--num-pages", type=int, default=None, help="pages in the pool (default: enough for every slot)")
    ap.add_argument("--max-num-seqs", type=int, default=8)
    ap.add_argument("--max-batched-tokens", type=int, default=2048)
    ap.add_argument("--prefill-chunk", type=int, default=256, help="longest prompt portion in one step (default 256)")
    ap.add_argument("--random-weights", type=int, metavar="SEED", default=None,
                    help="with --config: write a model folder with random weights from SEED (to -m, or a temporary folder) and use it")
    ap.add_argument("--config", help="config.json for --random-weights")
    ap.add_argument("--weights-dtype", default="float32", choices=["float32", "bfloat16"],
                    help="how --random-weights stores matrices (default float32)")
    return ap


def main(argv=None) -> int:
    args = build_parser().parse_args(argv)
    prompt = None
    if args.prompt_file:
        with open(args.prompt_file) as f:
            prompt = _ids(f.read())
    elif args.prompt is not None:
        prompt = _ids(args.prompt)
    if args.tokenize:
        if prompt is None:
            raise SystemExit("liyab-cli: --tokenize needs a prompt")
        print(" ".join(str(t) for t in prompt))
        return 0
    model_dir = args.model
    if args.random_weights is not None:
        if not args.config:
            raise SystemExit("liyab-cli: --random-weights needs --config")
        from .weights import write_random_model

        with open(args.config) as f:
            cfg = json.load(f)
        model_dir = model_dir or tempfile.mkdtemp(prefix="liyab-model-")
        write_random_model(model_dir, cfg, args.random_weights, dtype=args.weights_dtype)
        print(f"wrote {model_dir}", file=sys.stderr)
        if prompt is None:
            return 0
    if not model_dir:
        raise SystemExit("liyab-cli: -m MODEL is needed")
    if prompt is None:
        raise SystemExit("liyab-cli: -p PROMPT is needed")

    from . import Engine, SamplingParams
    from .errors import LiyabError

    t0 = time.perf_counter()
    try:
        engine = Engine(model_dir, dtype=args.dtype, device=args.device, page_size=args.page_size,
                        num_pages=args.num_pages, max_num_seqs=args.max_num_seqs,
                        max_batched_tokens=args.max_batched_tokens, prefill_chunk=args.prefill_chunk, ctx=args.ctx,
                        phases=args.phases)
        engine.warmup()  # kernels' code loaded here, not inside the first turn's time to first token
        engine.phases_ms(reset=True)
    except LiyabError as e:
        print(f"liyab-cli: {e}", file=sys.stderr)
        return 1
    load_ms = (time.perf_counter() - t0) * 1e3
    if args.json:
        print(json.dumps({"load_ms": round(load_ms, 3), "context": engine.core.max_positions,
                          "kv_cache_bytes_allocated": engine.core.storage.bytes_allocated(),
                          "dtype": str(engine.core.dtype).replace("torch.", "")}), flush=True)
    params = SamplingParams(temperature=args.temp, top_k=args.top_k, top_p=args.top_p, seed=args.seed, max_tokens=args.n)
    try:
        if args.json:
            res = engine.generate(prompt, params)
        else:
            def show(rid, token):
                print(token, end=" ", flush=True)
            res = engine.generate(prompt, params, on_token=show)
            print()
    except LiyabError as e:
        print(f"liyab-cli: {e}", file=sys.stderr)
        return 1
    s = res.stats
    phases = {k: round(v, 3) for k, v in engine.phases_ms().items()}
    if args.json:
        print(json.dumps({"turn": 0, **({"phases_ms": phases} if args.phases else {}), "prompt_tokens": s.prompt_tokens, "cached_prefix_tokens": 0,
                          "prefill_ms": round(s.prefill_ms, 3), "ttft_ms": round(s.ttft_ms, 3),
                          "generated_tokens": s.generated_tokens, "decode_ms": round(s.decode_ms, 3),
                          "tokens_per_second": round(s.tokens_per_second, 3), "kv_cache_bytes": s.kv_cache_bytes,
                          "finish_reason": res.finish_reason, "tokens": res.tokens}), flush=True)
    print(f"\n=== Generation ===\nprompt: {s.prompt_tokens} tokens (0 reused), {s.prefill_ms:.1f} ms, TTFT {s.ttft_ms:.1f} ms\n"
          f"decode: {s.generated_tokens} tokens, {s.decode_ms:.1f} ms, {s.tokens_per_second:.2f} tok/s\n"
          f"memory: KV {s.kv_cache_bytes / (1024.0 * 1024.0):.1f} MiB", file=sys.stderr)
    if phases:
        # as the reference prints them: device ms a generated token, phase by phase (tools/liyab_cli.cpp:198-211)
        per = max(1, s.generated_tokens)
        print("phases (ms/token): " + ", ".join(f"{k} {v / per:.3f}" for k, v in phases.items()), file=sys.stderr)
    return 0


if __name__ == "__main__":
    sys.exit(main())
