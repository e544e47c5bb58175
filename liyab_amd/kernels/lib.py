"""Loads the HIP kernel library and declares its entry points.

There is no fallback: if the library cannot be found, built or loaded, or
holds code for another GPU than the one present, importing fails with the
reason. The library is looked for where `csrc/build.py` puts it and built
on first use when it is not there.
"""

from __future__ import annotations

import ctypes
import struct
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


_EPI_PTR = ctypes.POINTER(EpiParams)
# which of the block's 8-byte words are addresses (a pointer field fills one word)
_EPI_ADDRESS_WORDS = [False] * ((ctypes.sizeof(EpiParams) + 7) // 8)
for _name, _type in EpiParams._fields_:
    if _type is P:
        _EPI_ADDRESS_WORDS[getattr(EpiParams, _name).offset // 8] = True
_EPI_ADDRESS_WORDS = tuple(_EPI_ADDRESS_WORDS)

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
    "liyab_gemm_mfma": [P, c_int64, P, c_int, c_int, c_int, c_int, _EPI_PTR, P],
    "liyab_gemm_mfma_dl": [P, c_int64, P, c_int, c_int, c_int, c_int, _EPI_PTR, P],
    "liyab_gemm_mfma_dl_parts": [P, c_int64, P, c_int, c_int, c_int, c_int, c_int, P, c_int64, P, P, c_int, c_int64, P],
    "liyab_gemm_skinny": [P, c_int64, P, c_int, c_int, c_int, c_int, c_int, c_int, _EPI_PTR, P],
    "liyab_attention_generic": [P, c_int64, P, c_int64, P, P, c_int, P, c_int, P, P, c_int, c_float, c_int, c_int,
                                c_int, c_int, c_int, c_int, P],
    "liyab_attention_decode": [P, c_int64, P, c_int64, P, P, c_int, P, c_int, P, P, P, c_int, c_float, c_int, c_int, c_int,
                               c_int, c_int, c_int, c_int, c_int, c_int, P, c_int, c_int, P],
    "liyab_attention_merge": [P, c_int, c_int64, P, c_int, c_int, c_int, c_int, P],
    "liyab_gemm_att_parts": [P, c_int, c_int, c_int, P, c_int, c_int, c_int, P, c_int64, P, P, c_int, c_int64, P],
    "liyab_gemm_skinny_ln": [P, c_int, c_int64, P, P, c_float, P, c_int, c_int, c_int, c_int, _EPI_PTR, P],
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
    for name, args in (("liyab_replay_index", [c_char_p, ctypes.POINTER(c_int)]),
                       ("liyab_replay", [ctypes.POINTER(ctypes.c_uint64), c_int64])):
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
    if _recording is not None:
        _record(name, args)


# -- a list of launches, recorded once and run again natively with other tensors ----------------
_recording: Optional[list] = None  # the words of the list being recorded, or None
_recording_addresses: Optional[list] = None  # for each of them: whether it is an address (a pointer argument or field)
_recording_whole = True  # whether every launch so far could be written down
_entries: dict = {}  # launcher name -> (index in the native table, encoders of its arguments)
BLOCK_ARG = 0xB10CB10CB10CB10C  # stands for the argument that points at an epilogue's parameter block (csrc/replay.hip)
_U64 = (1 << 64) - 1


def _encoders(name: str):
    """(index, [how each argument becomes a 64-bit word]) of a launcher the native replay knows,
    or None for one it does not."""
    hit = _entries.get(name)
    if hit is None:
        lib = load()
        n = c_int(0)
        index = lib.liyab_replay_index(name.encode(), ctypes.byref(n))
        kinds = []
        for t in _SIGNATURES[name]:
            kinds.append("block" if t is _EPI_PTR else "float" if t is c_float else "double" if t is c_double else
                         "address" if t is P else "int")
        hit = _entries[name] = (index, kinds) if index >= 0 and n.value == len(kinds) and "double" not in kinds else (-1, kinds)
    return hit


def _record(name: str, args) -> None:
    global _recording_whole
    index, kinds = _encoders(name)
    if index < 0:
        _recording_whole = False  # a launcher the native replay does not know: the list is of no use
        return
    words, addresses = [index, len(args)], [False, False]
    block, block_addresses = (), ()
    for kind, a in zip(kinds, args):
        addresses.append(kind == "address")
        if kind == "int" or kind == "address":
            words.append((0 if a is None else int(a)) & _U64)
        elif kind == "float":
            words.append(struct.unpack("<I", struct.pack("<f", a))[0])
        else:
            raw = bytes(a._obj)  # (the argument is ctypes.byref(params))
            raw += b"\0" * (-len(raw) % 8)
            block = struct.unpack(f"<{len(raw) // 8}Q", raw)
            block_addresses = _EPI_ADDRESS_WORDS
            words.append(BLOCK_ARG)
    words.append(len(block))
    words.extend(block)
    addresses.append(False)
    addresses.extend(block_addresses)
    _recording.extend(words)
    _recording_addresses.extend(addresses)


class recording:
    """Within this context every launch is also written down; `words` holds the list afterwards
    (a numpy array of uint64, see csrc/replay.hip) and `addresses` which of them are addresses
    (pointer arguments and pointer fields of a parameter block; a size or a constant never is), or
    None if a launcher ran that the native replay does not know."""

    def __enter__(self):
        global _recording, _recording_addresses, _recording_whole
        if _recording is not None:
            raise KernelError("a list of launches is being recorded already")
        _recording, _recording_addresses, _recording_whole = [], [], True
        self.words = self.addresses = None
        return self

    def __exit__(self, exc_type, *exc):
        global _recording, _recording_addresses
        import numpy as np

        words, _recording = _recording, None
        addresses, _recording_addresses = _recording_addresses, None
        if exc_type is None and _recording_whole:
            self.words = np.array(words, dtype=np.uint64)
            self.addresses = np.array(addresses, dtype=bool)
        return False


def replay(words) -> None:
    """Runs a recorded list of launches (a contiguous numpy array of uint64) again."""
    lib = load()
    rc = lib.liyab_replay(words.ctypes.data_as(ctypes.POINTER(ctypes.c_uint64)), words.size)
    if rc != 0:
        raise KernelError(f"replay: {lib.liyab_last_error().decode('utf-8', 'replace')}")
