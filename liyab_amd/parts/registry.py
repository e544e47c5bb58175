"""Registries from a spec's `kind` to the class that implements it.

The reference dispatches on `BlockPlan::mixer` and the feed-forward kind in
an if-chain inside `run_block` (src/compat/architecture.h:247-279,
src/core/transformer.cpp:5605-5637); here a new kind is one `register_*`
call, also from outside the package (a test registers a toy mixer so).
"""

from __future__ import annotations

from typing import Callable, Dict

from ..errors import Unsupported

_REGISTRIES: Dict[str, Dict[str, type]] = {
    "mixer": {}, "ffn": {}, "norm": {}, "position": {}, "block": {}, "embedding": {}, "head": {},
}


def _register(family: str, kind: str, cls: type) -> type:
    _REGISTRIES[family][kind] = cls
    return cls


def register_mixer(kind: str, cls: type) -> type: return _register("mixer", kind, cls)
def register_ffn(kind: str, cls: type) -> type: return _register("ffn", kind, cls)
def register_norm(kind: str, cls: type) -> type: return _register("norm", kind, cls)
def register_position(kind: str, cls: type) -> type: return _register("position", kind, cls)
def register_block(kind: str, cls: type) -> type: return _register("block", kind, cls)
def register_embedding(kind: str, cls: type) -> type: return _register("embedding", kind, cls)
def register_head(kind: str, cls: type) -> type: return _register("head", kind, cls)


def find_part(family: str, kind: str) -> type:
    reg = _REGISTRIES[family]
    if kind not in reg:
        raise Unsupported(f"{family} kind '{kind}' is not registered (registered: {','.join(sorted(reg)) or 'none'})")
    return reg[kind]


def build_part(family: str, spec, store, dtype):
    """The part for `spec` (by its `kind`), loading its tensors from `store`."""
    return find_part(family, spec.kind)(spec, store, dtype)
