"""From a model folder to a model on the device."""

from __future__ import annotations

import torch

from ..config.registry import load_config
from ..errors import InvalidArgument
from ..weights.loader import WeightStore
from .decoder import DecoderModel

DTYPES = {
    "bfloat16": torch.bfloat16, "bf16": torch.bfloat16,
    "float32": torch.float32, "fp32": torch.float32, "f32": torch.float32,
}


def resolve_dtype(dtype) -> torch.dtype:
    if isinstance(dtype, torch.dtype):
        if dtype not in (torch.float32, torch.bfloat16):
            raise InvalidArgument(f"dtype {dtype} is not one of bfloat16, float32")
        return dtype
    if dtype not in DTYPES:
        raise InvalidArgument(f"dtype '{dtype}' is not one of bfloat16, float32")
    return DTYPES[dtype]


def load_model(model_dir: str, dtype="bfloat16", device="cuda:0"):
    """(config, model): the class is chosen by config.json's architecture; all
    weight problems come as one InvalidModel."""
    config = load_config(model_dir)
    plan = config.plan()
    store = WeightStore.open(model_dir, device=device, compute_dtype=resolve_dtype(dtype),
                             name_prefixes=plan.name_prefixes, ignorable=plan.ignorable)
    model = DecoderModel(plan, store, resolve_dtype(dtype))
    store.finish()
    return config, model
