"""A small leveled logger for the engine's own messages.

The reference logs through a static ``Logger`` with ``init(app)``, ``info``,
``warning``, ``error`` and ``fatal`` that take printf formats
(src/log/Logger.h:17-36) on top of glog.  The same calls here, as functions of
this module, on top of nothing: one line per message on standard error,

    I1125 14:03:07.120 tffinfer] loaded /models/x in 2.1 s

with the level's letter first.  Messages below the threshold are dropped; the
threshold comes from ``set_level`` or the environment variable
``TFFINFER_LOG`` (debug, info, warning, error, fatal, off; default info).
``fatal`` logs and raises ``FatalError``; it does not end the process itself.
"""
from __future__ import annotations

import os
import sys
import threading
import time

DEBUG, INFO, WARNING, ERROR, FATAL, OFF = 10, 20, 30, 40, 50, 100
_NAMES = {"debug": DEBUG, "info": INFO, "warning": WARNING, "warn": WARNING, "error": ERROR,
          "fatal": FATAL, "off": OFF}
_LETTER = {DEBUG: "D", INFO: "I", WARNING: "W", ERROR: "E", FATAL: "F"}


class FatalError(RuntimeError):
    """Raised by ``fatal`` after the message is written."""


class _State:
    app = "tffinfer"
    level = INFO
    stream = None          # None: sys.stderr at the time of the call
    lock = threading.Lock()
    counts = {DEBUG: 0, INFO: 0, WARNING: 0, ERROR: 0, FATAL: 0}


def parse_level(name) -> int:
    if isinstance(name, int):
        return name
    try:
        return _NAMES[str(name).strip().lower()]
    except KeyError:
        raise ValueError(f"log level {name!r} is not one of {sorted(_NAMES)}") from None


def init(app_name: str = "tffinfer", level=None, stream=None) -> None:
    """Names the program in every line and sets the threshold (argument, else
    ``TFFINFER_LOG``, else info)."""
    _State.app = str(app_name)
    _State.stream = stream
    if level is None:
        level = os.environ.get("TFFINFER_LOG", "info")
    _State.level = parse_level(level)


def exit() -> None:
    """Flushes the stream (the reference shuts glog down here)."""
    s = _State.stream or sys.stderr
    try:
        s.flush()
    except (OSError, ValueError):
        pass


def set_level(level) -> None:
    _State.level = parse_level(level)


def get_level() -> int:
    return _State.level


def counts() -> dict:
    """Messages seen per level since the process began (dropped ones included)."""
    return {_LETTER[k]: v for k, v in _State.counts.items()}


def _emit(level: int, fmt: str, args) -> None:
    _State.counts[level] += 1
    if level < _State.level:
        return
    try:
        msg = fmt % args if args else fmt
    except (TypeError, ValueError):
        msg = f"{fmt} {args!r}"      # a message must never be lost to its own format
    t = time.time()
    lt = time.localtime(t)
    head = (f"{_LETTER[level]}{lt.tm_mon:02d}{lt.tm_mday:02d} {lt.tm_hour:02d}:{lt.tm_min:02d}:"
            f"{lt.tm_sec:02d}.{int(t * 1000) % 1000:03d} {_State.app}] ")
    s = _State.stream or sys.stderr
    with _State.lock:
        try:
            s.write(head + msg + "\n")
            s.flush()
        except (OSError, ValueError):
            pass


def debug(fmt: str, *args) -> None:
    _emit(DEBUG, fmt, args)


def info(fmt: str, *args) -> None:
    _emit(INFO, fmt, args)


def warning(fmt: str, *args) -> None:
    _emit(WARNING, fmt, args)


def error(fmt: str, *args) -> None:
    _emit(ERROR, fmt, args)


def fatal(fmt: str, *args) -> None:
    _emit(FATAL, fmt, args)
    raise FatalError(fmt % args if args else fmt)


if "TFFINFER_LOG" in os.environ:
    try:
        _State.level = parse_level(os.environ["TFFINFER_LOG"])
    except ValueError:
        pass
