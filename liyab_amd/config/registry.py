"""One registry from an architecture's name to its configuration class.

The reference keeps a table of registry rows and scans it by name
(`src/compat/architecture.cpp:415-426`); an unknown name is refused with the
list of the supported ones (`src/compat/architecture.cpp:578-585`). Here a
row is a configuration class with `from_json(dict)` and `plan()`; the model
itself is always the generic decoder built from the plan.
"""

from __future__ import annotations

import json
import os
from typing import Callable, Dict, List

from ..errors import InvalidModel, Unsupported

_ARCHITECTURES: Dict[str, type] = {}
_MODEL_TYPES: Dict[str, str] = {}


def register_architecture(name: str, config_cls: type, model_types: List[str] = ()) -> None:
    """Registers `config_cls` under config.json's `architectures[0]` name and,
    optionally, under `model_type` values that mean the same architecture."""
    _ARCHITECTURES[name] = config_cls
    for mt in model_types:
        _MODEL_TYPES[mt] = name


def supported_architectures() -> str:
    return ",".join(sorted(_ARCHITECTURES))


def find_architecture(name: str) -> type:
    cls = _ARCHITECTURES.get(name)
    if cls is None:
        raise Unsupported(
            f"architecture '{name}' is not supported yet (supported: {supported_architectures()})"
        )
    return cls


def architecture_name_of(raw: dict) -> str:
    archs = raw.get("architectures")
    if isinstance(archs, list) and archs and isinstance(archs[0], str):
        return archs[0]
    mt = raw.get("model_type")
    if isinstance(mt, str):
        if mt in _MODEL_TYPES:
            return _MODEL_TYPES[mt]
        raise Unsupported(
            f"architecture '{mt}' is not supported yet (supported: {supported_architectures()})"
        )
    raise InvalidModel("not a model folder: config.json has neither 'architectures' nor 'model_type'")


def config_from_dict(raw: dict):
    """Typed configuration for a parsed config.json."""
    if not isinstance(raw, dict):
        raise InvalidModel("config.json must hold a JSON object")
    return find_architecture(architecture_name_of(raw)).from_json(raw)


def load_config(model_dir: str):
    path = os.path.join(model_dir, "config.json")
    if not os.path.isfile(path):
        raise InvalidModel(f"not a model folder: '{path}' is missing")
    try:
        with open(path, "r", encoding="utf-8") as f:
            raw = json.load(f)
    except json.JSONDecodeError as e:
        raise InvalidModel(f"config.json is not valid JSON: {e}") from None
    return config_from_dict(raw)
