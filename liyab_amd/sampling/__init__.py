"""Sampling parameters, the per-token random numbers, and the device sampler.

Parameters and their defaults are the reference's `SamplingParams`
(include/liyab/types.h:215-222): temperature 0.8 (<= 0 is greedy), top_k 40
(<= 0 off), top_p 0.95 (>= 1 off), seed 0 = pick one at random, max_tokens
256. The order temperature -> top-k -> top-p -> renormalise -> draw is the
reference's (src/core/sampling.cpp:16-79) and runs in the sampling kernel.

The reference gives each generation its own `mt19937_64` (src/core/engine.cpp:3893),
which makes a request's draws independent of what else runs. Here the same
property comes from a counter-based generator: the uniform number for a
request's k-th generated token is a pure function of (seed, k), so it is
also the same after a preemption and recompute.
"""

from __future__ import annotations

import os
from dataclasses import dataclass
from typing import List, Optional, Sequence

_MASK = (1 << 64) - 1


@dataclass
class SamplingParams:
    temperature: float = 0.8
    top_k: int = 40
    top_p: float = 0.95
    seed: int = 0
    max_tokens: int = 256

    @property
    def greedy(self) -> bool:
        return not (self.temperature > 0.0)

    def resolved_seed(self) -> int:
        """The seed in use: a fresh random one when `seed` is 0."""
        if self.seed != 0:
            return self.seed & _MASK
        return int.from_bytes(os.urandom(8), "little") | 1


def uniform(seed: int, index: int) -> float:
    """A number in [0, 1) for token `index` of a request with `seed`:
    splitmix64's output function over a counter, top 53 bits."""
    z = (seed * 0x9E3779B97F4A7C15 + (index + 1) * 0xD1B54A32D192ED03) & _MASK
    z = (z + 0x9E3779B97F4A7C15) & _MASK
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _MASK
    z ^= z >> 31
    return (z >> 11) * (1.0 / (1 << 53))


class Sampler:
    """Samples one token per logits row on the device."""

    _RING = 4  # pinned staging buffers used in turn

    def __init__(self, device):
        import torch

        self.device = torch.device(device)
        self._cap = 0
        self._turn = 0

    def _buffers(self, rows: int):
        """Per-row parameters live in one device block, [uniform f64 | temperature f32 | top_k i32 |
        top_p f32] x capacity, filled from pinned host memory by one asynchronous copy a step."""
        import torch

        if rows > self._cap:
            cap = max(rows, 64, 2 * self._cap)
            self._out = torch.empty(cap, dtype=torch.int32, device=self.device)
            self._block = torch.empty(cap * 20, dtype=torch.uint8, device=self.device)
            self._u = self._block[:cap * 8].view(torch.float64)
            self._temp = self._block[cap * 8:cap * 12].view(torch.float32)
            self._topk = self._block[cap * 12:cap * 16].view(torch.int32)
            self._topp = self._block[cap * 16:cap * 20].view(torch.float32)
            self._host = [torch.empty(cap * 20, dtype=torch.uint8, pin_memory=True) for _ in range(self._RING)]
            self._host_np = [(h[:cap * 8].view(torch.float64).numpy(), h[cap * 8:cap * 12].view(torch.float32).numpy(),
                              h[cap * 12:cap * 16].view(torch.int32).numpy(), h[cap * 16:cap * 20].view(torch.float32).numpy())
                             for h in self._host]
            self._events = [None] * self._RING
            self._cap = cap

    def sample_on_device(self, logits, params: Sequence[SamplingParams], seeds: Sequence[int], indices: Sequence[int],
                         scatter=None, out=None):
        """One token per row of `logits` [rows, vocab] (float32, device), left on the device:
        returns an int32 tensor [rows] that stays valid until the next call. `seeds[r]` is row
        r's resolved seed and `indices[r]` how many tokens its request has generated so far.
        With scatter = (index, target), row r's token also goes to target[index[r]]. `out`: where
        the tokens go instead (int32, at least `rows` long; pinned host memory is taken: the kernel
        then writes the tokens where the host reads them once the stream has come that far)."""
        import torch

        from ..kernels import ops

        rows = logits.shape[0]
        if not (len(params) == len(seeds) == len(indices) == rows):
            raise ValueError("one SamplingParams, seed and index per logits row is needed")
        self._buffers(rows)
        out = self._out[:rows] if out is None else out[:rows]
        if all(p.greedy for p in params):
            ops.argmax(out, logits, scatter=scatter)
        else:
            i = self._turn
            self._turn = (i + 1) % self._RING
            if self._events[i] is not None:
                self._events[i].synchronize()  # its last copy has long finished
            u, temp, topk, topp = self._host_np[i]
            u[:rows] = [uniform(s, n) for s, n in zip(seeds, indices)]
            temp[:rows] = [p.temperature for p in params]
            topk[:rows] = [p.top_k for p in params]
            topp[:rows] = [p.top_p for p in params]
            self._block.copy_(self._host[i], non_blocking=True)
            if self._events[i] is None:
                self._events[i] = torch.cuda.Event()
            self._events[i].record()
            cuts = any(p.top_k > 0 or p.top_p < 1.0 for p in params)
            ops.sample(out, logits, self._temp[:rows], self._topk[:rows] if cuts else None,
                       self._topp[:rows] if cuts else None, self._u[:rows], scatter=scatter)
        return out

    def sample(self, logits, params: Sequence[SamplingParams], seeds: Sequence[int], indices: Sequence[int]) -> List[int]:
        """The same, with the tokens brought to the host."""
        return self.sample_on_device(logits, params, seeds, indices).tolist()
