"""Loads the HIP kernel library and declares its entry points.

There is no fallback: if the library cannot be found, built or loaded, or
holds code for another GPU than the one present, importing fails with the
reason. The library is looked for where `csrc/build.py` puts it and built
on first use when it is not there.
"""

from __future__ import annotations

import ctypes
import sys
from ctypes import c_char_p, c_double, c_float, c_int, c_int64, c_uint32, c_void_p
from typing import Optional

from ..csrc import build as _build
from ..errors import KernelError

_lib: Optional[ctypes.CDLL] = None
_path: Optional[str] = None

P = c_void_p


class EpiParams(ctypes.Structure):
    """Mirror of csrc/epilogue.h's EpiParams."""

    _fields_ = [
        ("mode", c_int), ("out_dtype", c_int), ("bias", P), ("out", P), ("ldo", c_int64), ("residual", P),
        ("ldr", c_int64), ("kc", P), ("vc", P), ("slots", P), ("q_dim", c_int), ("kv_dim", c_int), ("hd", c_int),
        ("n_kv_head", c_int), ("page_size", c_int), ("exact", c_int), ("num_slots", c_uint32),
    ]


_SIGNATURES = {
    "liyab_check_device": [],
    "liyab_fill": [P, c_int, c_uint32, c_int64, P],
    "liyab_add_into": [P, P, c_int, c_int64, P],
    "liyab_embed": [P, P, P, c_int, P, P, c_int, c_int, c_float, P, P],
    "liyab_add_rows": [P, P, c_int, P, c_int, c_int, P],
    "liyab_gather_rows": [P, c_int, P, P, c_int, c_int, P],
    "liyab_scale": [P, c_float, c_int64, P],
    "liyab_kv_write": [P, P, P, c_int, c_int64, c_int, c_int, P, c_int, c_int, c_int, c_int, c_int, P],
    "liyab_layernorm": [P, c_int, P, P, P, P, c_int, c_int, c_float, P],
    "liyab_layernorm_parts": [P, c_int, P, c_int, c_int64, c_int, P, P, P, c_int, c_int, c_float, P],
    "liyab_sum_parts": [P, c_int, c_int, P, c_int, c_int64, P],
    "liyab_gemm_skinny_parts": [P, c_int64, P, c_int, c_int, c_int, c_int, c_int, P, c_int64, P, P, c_int, c_int64, P],
    "liyab_gemm_simple": [P, c_int, c_int64, P, c_int64, P, c_int, P, P, c_int64, c_int, c_int, c_int, c_int, P],
    "liyab_gemm_mfma": [P, c_int64, P, c_int, c_int, c_int, c_int, ctypes.POINTER(EpiParams), P],
    "liyab_gemm_mfma_dl": [P, c_int64, P, c_int, c_int, c_int, c_int, ctypes.POINTER(EpiParams), P],
    "liyab_gemm_mfma_dl_parts": [P, c_int64, P, c_int, c_int, c_int, c_int, c_int, P, c_int64, P, P, c_int, c_int64, P],
    "liyab_gemm_skinny": [P, c_int64, P, c_int, c_int, c_int, c_int, c_int, c_int, ctypes.POINTER(EpiParams), P],
    "liyab_attention_generic": [P, c_int64, P, c_int64, P, P, c_int, P, c_int, P, P, c_int, c_float, c_int, c_int,
                                c_int, c_int, c_int, c_int, P],
    "liyab_attention_decode": [P, c_int64, P, c_int64, P, P, c_int, P, c_int, P, P, P, c_int, c_float, c_int, c_int, c_int,
                               c_int, c_int, c_int, c_int, c_int, c_int, P, c_int, c_int, P],
    "liyab_attention_merge": [P, c_int, c_int64, P, c_int, c_int, c_int, c_int, P],
    "liyab_gemm_att_parts": [P, c_int, c_int, c_int, P, c_int, c_int, c_int, P, c_int64, P, P, c_int, c_int64, P],
    "liyab_gemm_skinny_ln": [P, c_int, c_int64, P, P, c_float, P, c_int, c_int, c_int, c_int, ctypes.POINTER(EpiParams), P],
    "liyab_attention_prefill": [P, c_int64, P, c_int64, P, P, P, c_int, P, c_int, c_int, c_int, c_float, c_int, c_int,
                                c_int, c_int, c_int, c_int, P],
    "liyab_argmax": [P, P, c_int64, c_int, c_int, P, P, P, P, P],
    "liyab_argmax_static_init": [],
    "liyab_argmax_static": [P, P, c_int64, c_int, c_int, P, P, P],
    "liyab_sample": [P, P, c_int64, c_int, c_int, P, P, P, P, P, P, P],
}


def library_path() -> Optional[str]:
    return _path


def load() -> ctypes.CDLL:
    """The loaded library; builds it first when no built library exists."""
    global _lib, _path
    if _lib is not None:
        return _lib
    path = _build.find_library()
    if path is None:
        try:
            path = _build.build()
        except Exception as e:  # noqa: BLE001
            raise KernelError(f"the HIP kernel library is not built and building it failed: {e}") from e
    elif _build.is_stale(path):
        # built from other sources than those in csrc/: never serve them silently
        print(f"[liyab_amd] {path} was built from other sources than those in csrc/: building it again",
              file=sys.stderr, flush=True)
        try:
            path = _build.build()
        except Exception as e:  # noqa: BLE001
            raise KernelError(f"the HIP kernel library is stale and building it again failed: {e}") from e
    try:
        lib = ctypes.CDLL(path)
    except OSError as e:
        raise KernelError(f"cannot load the HIP kernel library '{path}': {e}") from e
    lib.liyab_last_error.restype = c_char_p
    lib.liyab_last_error.argtypes = []
    for name, args in _SIGNATURES.items():
        fn = getattr(lib, name, None)
        if fn is None:
            raise KernelError(f"'{path}' lacks the entry point {name}: rebuild it (python -m liyab_amd.csrc.build)")
        fn.restype = c_int
        fn.argtypes = args
    _lib, _path = lib, path
    return lib


def call(name: str, *args) -> None:
    lib = load()
    rc = getattr(lib, name)(*args)
    if rc != 0:
        raise KernelError(f"{name}: {lib.liyab_last_error().decode('utf-8', 'replace')}")
