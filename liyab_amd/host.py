"""The binding to the host library (`csrc/host/`: cache manager, step metadata).

Loaded through ctypes; built with the system's C++ compiler on first use when no
library built from the current sources is found (a few seconds). It is plain C++
without any HIP in it, so it loads and runs where there is no GPU.
"""

from __future__ import annotations

import ctypes
from ctypes import POINTER, c_char_p, c_int, c_int32, c_int64, c_void_p

from .errors import Busy, ContextFull, InvalidArgument, OutOfPages

MAX_GROUPS = 16


class StepShape(ctypes.Structure):
    """Mirror of liyab_host::StepShape (csrc/host/step_meta.h)."""

    _fields_ = [(n, c_int) for n in (
        "n_tokens", "n_rows", "n_seqs", "n_logit_rows", "n_groups", "max_blocks", "max_q_len",
        "max_context", "total", "off_token_ids", "off_positions", "off_tok_seq", "off_seq_starts", "off_context_lens",
        "off_state_slots", "off_logit_rows", "off_logit_slots")] + [
        ("off_block_tables", c_int * MAX_GROUPS), ("off_slots", c_int * MAX_GROUPS)]


class Scheduled(ctypes.Structure):
    """Mirror of liyab_host::Scheduled (csrc/host/scheduler.h)."""

    _fields_ = [(n, c_int) for n in ("id", "slot", "first", "count", "wants_logits")]


IP = POINTER(c_int)
_SIGNATURES = {
    "liyab_host_last_error": ([], c_char_p),
    "liyab_pool_create": ([c_int], c_void_p),
    "liyab_pool_destroy": ([c_void_p], None),
    "liyab_pool_allocate": ([c_void_p, c_int, POINTER(c_int32)], c_int),
    "liyab_pool_release": ([c_void_p, POINTER(c_int32), c_int], c_int),
    "liyab_pool_check": ([c_void_p], c_int),
    "liyab_pool_free_pages": ([c_void_p], c_int),
    "liyab_pool_peak": ([c_void_p], c_int),
    "liyab_cm_create": ([c_int, IP, IP, c_int, c_int, c_int], c_void_p),
    "liyab_cm_destroy": ([c_void_p], None),
    "liyab_cm_open": ([c_void_p, IP], c_int),
    "liyab_cm_close": ([c_void_p, c_int], c_int),
    "liyab_cm_length": ([c_void_p, c_int], c_int),
    "liyab_cm_pages_needed": ([c_void_p, c_int, c_int, IP], None),
    "liyab_cm_reserve": ([c_void_p, IP, IP, c_int], c_int),
    "liyab_cm_reserve_more": ([c_void_p, IP, IP, c_int, IP], c_int),
    "liyab_cm_commit": ([c_void_p, c_int, c_int], c_int),
    "liyab_cm_commit_many": ([c_void_p, IP, IP, c_int], c_int),
    "liyab_cm_truncate": ([c_void_p, c_int, c_int], c_int),
    "liyab_cm_table_rows": ([c_void_p, c_int], POINTER(c_int32)),
    "liyab_cm_table_length": ([c_void_p, c_int, c_int], c_int),
    "liyab_cm_max_blocks": ([c_void_p], c_int),
    "liyab_cm_free_slots": ([c_void_p], c_int),
    "liyab_cm_free_pages": ([c_void_p, c_int], c_int),
    "liyab_cm_peak_in_use": ([c_void_p, c_int], c_int),
    "liyab_cm_check": ([c_void_p], c_int),
    "liyab_sched_create": ([c_void_p, c_int, c_int, c_int], c_void_p),
    "liyab_sched_destroy": ([c_void_p], None),
    "liyab_sched_add": ([c_void_p, c_int, c_int, c_int, IP], c_int),
    "liyab_sched_pressure": ([c_void_p], c_int),
    "liyab_sched_schedule": ([c_void_p, POINTER(POINTER(Scheduled)), POINTER(IP), POINTER(IP), IP], c_int),
    "liyab_sched_advance": ([c_void_p, POINTER(Scheduled), c_int], None),
    "liyab_sched_tokens": ([c_void_p, IP, IP, c_int, IP], None),
    "liyab_sched_finish": ([c_void_p, c_int], c_int),
    "liyab_sched_get": ([c_void_p, c_int, c_int], c_int),
    "liyab_sched_list": ([c_void_p, c_int, IP, c_int], c_int),
    "liyab_sched_stats": ([c_void_p, POINTER(ctypes.c_longlong)], None),
    "liyab_step_shape": ([c_void_p, c_int, IP, IP, IP, c_int, POINTER(StepShape)], c_int),
    "liyab_step_fill": ([c_void_p, POINTER(StepShape), IP, IP, POINTER(c_int64), IP, IP, c_int, POINTER(c_int32)], c_int),
    "liyab_attn_counts": ([c_int, IP, c_int, c_int, IP], None),
    "liyab_attn_fill": ([c_int, IP, IP, c_int, c_int, POINTER(c_int32)], None),
}

_lib = None

# Status codes of the library (csrc/host/cache_manager.h) and what they become here
_ERRORS = {1: InvalidArgument, 2: OutOfPages, 3: ContextFull, 4: Busy, 5: AssertionError}


def lib():
    """The loaded library; builds it first when none fits the current sources."""
    global _lib
    if _lib is None:
        from .csrc import build

        path = build.find_host_library() or build.build_host()
        loaded = ctypes.CDLL(path)
        for name, (args, res) in _SIGNATURES.items():
            fn = getattr(loaded, name)
            fn.argtypes, fn.restype = args, res
        _lib = loaded
    return _lib


def check(status: int) -> None:
    """Raises the error a non-zero status stands for, with the library's message."""
    if status:
        raise _ERRORS.get(status, AssertionError)(lib().liyab_host_last_error().decode())
