"""One place that decides what the package says on stderr.

``LYAPUNOV_AMD_LOG`` = ``quiet`` (warnings only), ``info`` (the default: also
progress lines of builds and warm-ups) or ``debug`` (also counters when an
engine is dropped); ``set_level`` does the same from code.  The reference's
logger has the same ladder with time stamps
(csrc/include/utils/logging.hpp:30-73: DEBUG < INFO < WARNING < ERROR, a level
below the current one is not printed); errors here are exceptions, not lines.
"""
from __future__ import annotations

import os
import sys

LEVELS = {"debug": 0, "info": 1, "quiet": 2}
_PREFIX = "[lyapunov-amd]"


def _from_env() -> int:
    name = os.environ.get("LYAPUNOV_AMD_LOG", "info").strip().lower()
    if name not in LEVELS:
        raise ValueError(f"LYAPUNOV_AMD_LOG is one of {sorted(LEVELS)}, not {name!r}")
    return LEVELS[name]


_level = _from_env()


def set_level(name: str) -> None:
    global _level
    if name not in LEVELS:
        raise ValueError(f"a log level is one of {sorted(LEVELS)}, not {name!r}")
    _level = LEVELS[name]


def level() -> str:
    return next(k for k, v in LEVELS.items() if v == _level)


def _say(msg: str, prefix: str = _PREFIX) -> None:
    print(f"{prefix} {msg}", file=sys.stderr, flush=True)


def debug(msg: str) -> None:
    if _level <= LEVELS["debug"]:
        _say(msg)


def info(msg: str, prefix: str = _PREFIX) -> None:
    if _level <= LEVELS["info"]:
        _say(msg, prefix)


def warn(msg: str) -> None:
    """Something was switched off or ignored: said at every level."""
    _say(msg)


__all__ = ["set_level", "level", "debug", "info", "warn", "LEVELS"]
