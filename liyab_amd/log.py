"""Log lines of the engine, in the manner of the reference's LIYAB_LOG_{DEBUG,INFO,WARN,ERROR}
(src/core/log.h:14-34): a level, a printf-style message, an optional sink. The level comes from
the environment variable LIYAB_LOG (debug, info, warn, error; default warn), as the reference's
does (docs/guide/development.md:35); `set_sink` sends lines elsewhere than standard error."""

from __future__ import annotations

import os
import sys
from typing import Callable, Optional

LEVELS = {"debug": 0, "info": 1, "warn": 2, "error": 3}
_level = LEVELS.get(os.environ.get("LIYAB_LOG", "warn").strip().lower(), 2)
_sink: Optional[Callable[[str, str], None]] = None


def set_level(name: str) -> None:
    global _level
    if name not in LEVELS:
        raise ValueError(f"log level '{name}' is not one of {', '.join(LEVELS)}")
    _level = LEVELS[name]


def set_sink(sink: Optional[Callable[[str, str], None]]) -> None:
    """`sink(level, line)` receives every line at or above the level; None: standard error."""
    global _sink
    _sink = sink


def _emit(level: str, fmt: str, args) -> None:
    if LEVELS[level] < _level:
        return
    line = fmt % args if args else fmt
    if _sink is not None:
        _sink(level, line)
    else:
        print(f"[liyab_amd {level}] {line}", file=sys.stderr, flush=True)


def debug(fmt: str, *args) -> None: _emit("debug", fmt, args)
def info(fmt: str, *args) -> None: _emit("info", fmt, args)
def warn(fmt: str, *args) -> None: _emit("warn", fmt, args)
def error(fmt: str, *args) -> None: _emit("error", fmt, args)
