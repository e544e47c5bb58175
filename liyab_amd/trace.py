"""Trace replay: given token ids, step by step, logits out. Samples nothing.

It drives the engine's own model, step function, cache and kernels -- the
ones generation uses -- through `EngineCore.step`. The reference's nearest
tools feed a text through the model in passes and compare per-position
outputs (`tools/liyab_kl.cpp:1-30`; teacher-forced per-position records in
`tools/conform_reference.py:166-180`) and replay plans of prompt portions
and decoding steps through forward and forward_batch
(`tests/test_sequences.cpp:82-238`).

    trace_run --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N

Standard input holds one JSON object a line:
    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}
All entries of a step are one batch. For a step in which something is
wanted, `OUT/<step>.f32` holds the logits at the wanted places as
little-endian float32 [wanted, vocab], in the order of the entries and of
`want`. After every step a line `done <step>` is printed and flushed.
"""

from __future__ import annotations

import argparse
import json
import os
import sys


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", required=True, choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True, help="folder the logits files are written to")
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="the most tokens live requests hold at any time (each rounded up to a multiple of 64)")
    ap.add_argument("--page-size", type=int, default=16, help="tokens per cache page (default 16; must divide 64)")
    ap.add_argument("--device", default="cuda:0")
    args = ap.parse_args(argv)
    if args.max_tokens <= 0:
        ap.error("--max-tokens must be positive")
    if args.page_size <= 0 or 64 % args.page_size != 0:
        ap.error("--page-size must divide 64")
    os.makedirs(args.out, exist_ok=True)

    from .kernels import load as load_kernels

    load_kernels()  # builds the library on a first call in a fresh checkout; prints progress
    import numpy as np

    from .engine import EngineCore, StepItem

    core = EngineCore(args.model, dtype=args.dtype, device=args.device, page_size=args.page_size,
                      max_tokens=args.max_tokens, max_requests=16)
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        rec = json.loads(line)
        step = rec["step"]
        items = []
        for e in rec.get("entries", []):
            rid = e["id"]
            if not core.is_open(rid):
                core.open(rid)
            items.append(StepItem(rid=rid, tokens=e["tokens"], want=e.get("want", [])))
        if items:
            logits = core.step(items)
            if logits is not None:
                arr = logits.to("cpu").numpy().astype("<f4", copy=False)
                tmp = os.path.join(args.out, f".{step}.f32.tmp")
                arr.tofile(tmp)
                os.replace(tmp, os.path.join(args.out, f"{step}.f32"))
        for rid in rec.get("end", []):
            if core.is_open(rid):
                core.close(rid)
        print(f"done {step}", flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
