"""What the C library over the engine calls (`csrc/capi/liyab_engine_c.cpp`).

`libliyab_engine.so` runs these two functions in a Python interpreter inside the C program's
process: `create` for `liyab_engine_create`, `generate` for `liyab_engine_generate_tokens`
(the reference's C ABI, include/liyab/liyab_c_api.h:223-252). Arguments and results are plain
numbers, strings and bytes, so that the C side needs nothing of this package's types.
"""

from __future__ import annotations

import ctypes
import struct

from .engine import Engine
from .sampling import SamplingParams

_CALLBACK = ctypes.CFUNCTYPE(ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p)


def create(model_path: str, dtype: str, context_length: int, page_size: int, num_pages: int, max_sequences: int,
           max_batched_tokens: int, prefill_chunk: int, batch_invariant: int) -> Engine:
    engine = Engine(model_path, dtype=dtype, ctx=context_length or None, page_size=page_size, num_pages=num_pages or None,
                    max_num_seqs=max_sequences, max_batched_tokens=max_batched_tokens, prefill_chunk=prefill_chunk,
                    batch_invariant=bool(batch_invariant))
    engine.warmup()
    return engine


def generate(engine: Engine, prompt: bytes, temperature: float, top_k: int, top_p: float, seed: int, max_tokens: int,
             callback: int, user_data: int):
    """Blocking generation; returns (generated ids as bytes of int32, prompt_tokens, prefill_ms,
    ttft_ms, decode_ms, tokens_per_second, kv_cache_bytes, preemptions, cancelled)."""
    ids = list(struct.unpack(f"<{len(prompt) // 4}i", prompt))
    params = SamplingParams(temperature=temperature, top_k=top_k, top_p=top_p, seed=seed, max_tokens=max_tokens)
    on_token = None
    if callback:
        fn = _CALLBACK(callback)
        on_token = lambda rid, token: bool(fn(int(token), user_data or None))  # noqa: E731
    res = engine.generate(ids, params, on_token=on_token)
    s = res.stats
    out = struct.pack(f"<{len(res.tokens)}i", *res.tokens)
    return (out, s.prompt_tokens, s.prefill_ms, s.ttft_ms, s.decode_ms, s.tokens_per_second, int(s.kv_cache_bytes),
            int(s.preemptions), int(res.finish_reason == "callback"))
