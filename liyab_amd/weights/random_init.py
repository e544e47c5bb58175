"""Random-weights mode: a model folder from a configuration and a seed.

The role of the reference's `tools/tiny_checkpoint.py` (a checkpoint of an
architecture with random weights, `:1-14`) and of its test writer
`write_tiny_model` (`tests/test_model.cpp:603-647`: matrices, norm weights
near 1 and biases from seeded generators). The distributions here are those
the benchmark configurations name: embeddings and linear weights N(0, 0.02),
the two output projections N(0, 0.02 / sqrt(2 n_layer)), biases N(0, 0.02),
norm weights 1 + N(0, 0.05), norm biases N(0, 0.02). Norm weights away from
1 and non-zero biases make a norm or bias applied in the wrong place visible
(`tools/reference_trace.py:424-437` argues the same).

The tensors are drawn in the order the plan lists them, each from its own
generator seeded by (seed, index), so a tensor's values do not depend on the
sizes of the others.
"""

from __future__ import annotations

import json
import math
import os
from typing import Dict

import numpy as np
import torch

from ..config.gpt2 import GPT2Config
from .loader import WEIGHTS_FILE
from .safetensors_io import write_safetensors


def _normal(seed: int, index: int, shape, std: float, mean: float = 0.0) -> torch.Tensor:
    rng = np.random.Generator(np.random.Philox(key=[seed & 0xFFFFFFFFFFFFFFFF, index]))
    a = rng.standard_normal(size=shape, dtype=np.float32)
    return torch.from_numpy(a * np.float32(std) + np.float32(mean))


def random_gpt2_tensors(cfg: GPT2Config, seed: int) -> Dict[str, torch.Tensor]:
    """float32 tensors under GPT-2's checkpoint names and stored layouts
    (the four projection matrices are stored [in, out])."""
    d, F = cfg.n_embd, cfg.n_inner
    proj_std = 0.02 / math.sqrt(2.0 * cfg.n_layer)
    out: Dict[str, torch.Tensor] = {}
    idx = 0

    def add(name, shape, std, mean=0.0):
        nonlocal idx
        out[name] = _normal(seed, idx, shape, std, mean)
        idx += 1

    add("wte.weight", (cfg.vocab_size, d), 0.02)
    add("wpe.weight", (cfg.n_positions, d), 0.02)
    for i in range(cfg.n_layer):
        p = f"h.{i}"
        add(p + ".ln_1.weight", (d,), 0.05, 1.0)
        add(p + ".ln_1.bias", (d,), 0.02)
        add(p + ".attn.c_attn.weight", (d, 3 * d), 0.02)
        add(p + ".attn.c_attn.bias", (3 * d,), 0.02)
        add(p + ".attn.c_proj.weight", (d, d), proj_std)
        add(p + ".attn.c_proj.bias", (d,), 0.02)
        add(p + ".ln_2.weight", (d,), 0.05, 1.0)
        add(p + ".ln_2.bias", (d,), 0.02)
        add(p + ".mlp.c_fc.weight", (d, F), 0.02)
        add(p + ".mlp.c_fc.bias", (F,), 0.02)
        add(p + ".mlp.c_proj.weight", (F, d), proj_std)
        add(p + ".mlp.c_proj.bias", (d,), 0.02)
    add("ln_f.weight", (d,), 0.05, 1.0)
    add("ln_f.bias", (d,), 0.02)
    if not cfg.tie_word_embeddings:
        add("lm_head.weight", (cfg.vocab_size, d), 0.02)
    return out


_GENERATORS = {"GPT2LMHeadModel": random_gpt2_tensors}


def write_random_model(out_dir: str, config: dict | GPT2Config, seed: int, dtype: str = "float32") -> str:
    """Writes `out_dir/config.json` and `out_dir/model.safetensors`.

    `dtype` is how matrices are stored: "float32" or "bfloat16" (vectors are
    always float32). Returns `out_dir`."""
    from ..config.registry import config_from_dict

    cfg = config if not isinstance(config, dict) else config_from_dict(config)
    gen = _GENERATORS.get(cfg.architecture)
    if gen is None:
        raise KeyError(f"no random-weights generator for architecture '{cfg.architecture}'")
    if dtype not in ("float32", "bfloat16"):
        raise ValueError("dtype must be 'float32' or 'bfloat16'")
    tensors = gen(cfg, int(seed))
    if dtype == "bfloat16":
        tensors = {k: (v.to(torch.bfloat16) if v.dim() >= 2 else v) for k, v in tensors.items()}
    os.makedirs(out_dir, exist_ok=True)
    raw = cfg.to_json()
    raw["dtype"] = dtype
    with open(os.path.join(out_dir, "config.json"), "w", encoding="utf-8") as f:
        json.dump(raw, f, indent=1)
    write_safetensors(os.path.join(out_dir, WEIGHTS_FILE), tensors, {"format": "pt", "seed": str(seed)})
    return out_dir
