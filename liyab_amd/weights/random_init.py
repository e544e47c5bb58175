"""Random-weights mode: a model folder from a configuration and a seed.

The role of the reference's `tools/tiny_checkpoint.py` (a checkpoint of an
architecture with random weights, `:1-14`) and of its test writer
`write_tiny_model` (`tests/test_model.cpp:603-647`: matrices, norm weights
near 1 and biases from seeded generators).

Nothing here knows an architecture. The tensors are those the model's parts
ask for when the model is built from its plan: the build runs against a
store that draws each tensor it is asked for, in the shape the part expects
and the layout the plan says the file holds, from the distribution the plan
gives with the tensor's name (`TensorSource.init`; N(0, 0.02) where the plan
says nothing). So a new architecture, or a toy one made of parts a test
registers, gets its random-weights mode from its plan alone.

Each tensor has a generator of its own, keyed by the seed and the tensor's
name: its values depend neither on the other tensors' sizes nor on the order
in which parts are built.
"""

from __future__ import annotations

import json
import os
from typing import Dict, Optional, Sequence

import numpy as np
import torch

from ..config.plan import Init, TensorSource
from .loader import WEIGHTS_FILE
from .safetensors_io import write_safetensors

DEFAULT_INIT = Init(std=0.02)


def _name_key(name: str) -> int:
    """FNV-1a over the name's bytes, 64 bits: the same on every machine and run."""
    h = 0xCBF29CE484222325
    for b in name.encode("utf-8"):
        h = ((h ^ b) * 0x100000001B3) & 0xFFFFFFFFFFFFFFFF
    return h


def draw(seed: int, name: str, shape: Sequence[int], init: Init) -> torch.Tensor:
    """float32 N(init.mean, init.std) of `shape` from the generator of (seed, name)."""
    rng = np.random.Generator(np.random.Philox(key=[seed & 0xFFFFFFFFFFFFFFFF, _name_key(name)]))
    a = rng.standard_normal(size=tuple(int(s) for s in shape), dtype=np.float32)
    return torch.from_numpy(a * np.float32(init.std) + np.float32(init.mean))


class DrawingStore:
    """Stands where a `WeightStore` stands while a model is built, and draws what it is asked
    for. `tensors` ends up holding every tensor under its file name, in its stored layout."""

    def __init__(self, seed: int):
        self.seed = int(seed)
        self.tensors: Dict[str, torch.Tensor] = {}
        self.device = torch.device("cpu")
        self.compute_dtype = torch.float32

    def has(self, src: TensorSource) -> bool:
        return src.required or src.name in self.tensors

    def fetch(self, src: TensorSource, shape: Sequence[int], role: str) -> Optional[torch.Tensor]:
        if not src.required and src.name not in self.tensors:
            return None  # an optional tensor stays absent
        shape = tuple(int(s) for s in shape)
        stored = (shape[1], shape[0]) if src.layout == "in_out" else shape
        t = self.tensors.get(src.name)
        if t is None:
            if role == "index":
                raise ValueError(f"random weights: no rule for the integer tensor '{src.name}'")
            t = self.tensors[src.name] = draw(self.seed, src.name, stored, src.init or DEFAULT_INIT)
        elif tuple(t.shape) != stored:
            raise ValueError(f"random weights: '{src.name}' is asked for as {list(stored)} and as {list(t.shape)}")
        return t.t() if src.layout == "in_out" else t

    def finish(self) -> None:
        pass


def random_tensors(config, seed: int) -> Dict[str, torch.Tensor]:
    """float32 tensors under the file names and in the stored layouts of `config`'s plan (a
    typed configuration, or a `ModelPlan`)."""
    from ..models.decoder import DecoderModel

    plan = config.plan() if hasattr(config, "plan") else config
    store = DrawingStore(seed)
    DecoderModel(plan, store, torch.float32)
    return store.tensors


def write_random_model(out_dir: str, config, seed: int, dtype: str = "float32") -> str:
    """Writes `out_dir/config.json` and `out_dir/model.safetensors` for a configuration (a
    config.json dict, or the typed configuration of any registered architecture).

    `dtype` is how matrices are stored: "float32" or "bfloat16" (vectors are
    always float32). Returns `out_dir`."""
    from ..config.registry import config_from_dict

    cfg = config if not isinstance(config, dict) else config_from_dict(config)
    if dtype not in ("float32", "bfloat16"):
        raise ValueError("dtype must be 'float32' or 'bfloat16'")
    tensors = random_tensors(cfg, int(seed))
    if dtype == "bfloat16":
        tensors = {k: (v.to(torch.bfloat16) if v.dim() >= 2 else v) for k, v in tensors.items()}
    os.makedirs(out_dir, exist_ok=True)
    raw = cfg.to_json()
    raw["dtype"] = dtype
    with open(os.path.join(out_dir, "config.json"), "w", encoding="utf-8") as f:
        json.dump(raw, f, indent=1)
    write_safetensors(os.path.join(out_dir, WEIGHTS_FILE), tensors, {"format": "pt", "seed": str(seed)})
    return out_dir
