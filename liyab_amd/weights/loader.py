"""Weights by tensor name, with one error that says everything wrong.

Parts ask the store for their tensors by the names the plan gives them, with
the shape they expect. The reference binds each tensor the same way and
refuses with "missing tensor 'N'" or "tensor 'N' has shape [...], expected
[...]" (`src/core/transformer.cpp:1052-1072`), one failure at a time; here
every problem is collected and `finish()` raises a single `InvalidModel`
that lists missing tensors, wrong shapes and names nobody asked for.

Precision: matrices and tables go to the device in the compute dtype of the
path (bfloat16 for serving, float32 for the 32-bit path); vectors (norm
weights, biases) are float32 on both paths; integer tensors become int32.
A tensor is converted once, at load, and stays resident.
"""

from __future__ import annotations

import fnmatch
import os
from typing import Dict, List, Optional, Sequence, Tuple

import torch

from ..config.plan import TensorSource
from ..errors import InvalidModel
from .safetensors_io import SafetensorsFile

WEIGHTS_FILE = "model.safetensors"


class WeightStore:
    def __init__(
        self,
        tensors: Dict[str, torch.Tensor],
        *,
        device: torch.device | str,
        compute_dtype: torch.dtype,
        name_prefixes: Sequence[str] = ("",),
        ignorable: Sequence[str] = (),
        origin: str = "<memory>",
    ):
        self._tensors = tensors
        self.device = torch.device(device)
        self.compute_dtype = compute_dtype
        self._prefixes = tuple(name_prefixes) or ("",)
        self._ignorable = tuple(ignorable)
        self.origin = origin
        self._used: set = set()
        self._missing: List[str] = []
        self._wrong: List[str] = []
        self._cache: Dict[Tuple[str, str, str], torch.Tensor] = {}

    # -- construction -----------------------------------------------------
    @classmethod
    def open(cls, model_dir: str, **kw) -> "WeightStore":
        path = os.path.join(model_dir, WEIGHTS_FILE)
        f = SafetensorsFile(path)
        tensors = {name: f.tensor(name) for name in f.entries}
        store = cls(tensors, origin=path, **kw)
        store._file = f
        return store

    # -- lookup -----------------------------------------------------------
    def _resolve(self, name: str) -> Optional[str]:
        for p in self._prefixes:
            if p + name in self._tensors:
                return p + name
        return None

    def has(self, src: TensorSource) -> bool:
        return self._resolve(src.name) is not None

    def fetch(self, src: TensorSource, shape: Sequence[int], role: str) -> Optional[torch.Tensor]:
        """The tensor `src` names, on the device, in working layout and dtype.

        `shape` is the working shape ("out_in" for matrices); `role` is
        "matrix" or "table" (compute dtype), "vector" (float32) or "index"
        (int32). A problem is recorded and a zero tensor of the right shape
        returned, so that loading goes on and finds the others; `finish()`
        raises. An optional tensor that is absent gives None.
        """
        shape = tuple(int(s) for s in shape)
        full = self._resolve(src.name)
        if full is None:
            if not src.required:
                return None
            self._missing.append(src.name)
            return self._placeholder(shape, role)
        self._used.add(full)
        key = (full, src.layout, role)
        if key in self._cache:
            return self._cache[key]
        t = self._tensors[full]
        stored_shape = tuple(t.shape)
        want_stored = shape
        if src.layout == "in_out":
            if len(shape) != 2:
                raise ValueError("layout 'in_out' is for matrices")
            want_stored = (shape[1], shape[0])
        if stored_shape != want_stored:
            self._wrong.append(
                f"tensor '{src.name}' has shape {list(stored_shape)}, expected {list(want_stored)}"
            )
            return self._placeholder(shape, role)
        dtype = self._dtype_for(role, t.dtype, src.name)
        if dtype is None:
            return self._placeholder(shape, role)
        dev = t.to(self.device, copy=True)
        if src.layout == "in_out":
            dev = dev.t()
        dev = dev.to(dtype).contiguous()
        self._cache[key] = dev
        return dev

    def _dtype_for(self, role: str, stored: torch.dtype, name: str) -> Optional[torch.dtype]:
        if role == "index":
            if stored.is_floating_point:
                self._wrong.append(f"tensor '{name}' holds {stored}, expected integers")
                return None
            return torch.int32
        if not stored.is_floating_point:
            self._wrong.append(f"tensor '{name}' holds {stored}, expected floating point")
            return None
        return torch.float32 if role == "vector" else self.compute_dtype

    def _placeholder(self, shape, role) -> torch.Tensor:
        dtype = {"vector": torch.float32, "index": torch.int32}.get(role, self.compute_dtype)
        return torch.zeros(shape, dtype=dtype, device=self.device)

    # -- the one error ----------------------------------------------------
    def unexpected(self) -> List[str]:
        out = []
        for name in self._tensors:
            if name in self._used:
                continue
            bare = name
            for p in self._prefixes:
                if p and name.startswith(p):
                    bare = name[len(p):]
                    break
            if any(fnmatch.fnmatchcase(bare, pat) or fnmatch.fnmatchcase(name, pat) for pat in self._ignorable):
                continue
            out.append(name)
        return out

    def finish(self) -> None:
        """Raises one InvalidModel naming every missing, mis-shaped and
        unexpected tensor, or returns when there is none."""
        unexpected = self.unexpected()
        if not (self._missing or self._wrong or unexpected):
            return
        lines = [f"the weights in '{self.origin}' do not fit the configuration:"]
        if self._missing:
            lines.append(f"  missing tensors ({len(self._missing)}): " + ", ".join(f"'{n}'" for n in self._missing))
        if self._wrong:
            lines.append(f"  wrong shapes or types ({len(self._wrong)}):")
            lines.extend("    " + w for w in self._wrong)
        if unexpected:
            lines.append(f"  unexpected tensors ({len(unexpected)}): " + ", ".join(f"'{n}'" for n in unexpected))
        raise InvalidModel("\n".join(lines))
