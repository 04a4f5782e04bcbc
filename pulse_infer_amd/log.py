"""Messages with a level: trace, debug, info, warn, error, fatal, and ``set_level`` / ``set_pattern``
(reference: include/pulse/logging.hpp:13-130, the same six calls over spdlog).  Everything goes to
standard error under the name of the package, so that what a program prints on standard output (token ids,
``done <step>`` lines, a benchmark's JSON) stays clean.  The level comes from ``PULSE_LOG_LEVEL``
(trace, debug, info, warn, error, critical, off; default info) until ``set_level`` says otherwise.
"""
from __future__ import annotations

import logging as _logging
import os
import sys

TRACE = 5
LEVELS = {"trace": TRACE, "debug": _logging.DEBUG, "info": _logging.INFO, "warn": _logging.WARNING,
          "warning": _logging.WARNING, "error": _logging.ERROR, "err": _logging.ERROR,
          "critical": _logging.CRITICAL, "fatal": _logging.CRITICAL, "off": _logging.CRITICAL + 10}
DEFAULT_PATTERN = "[pulse_infer_amd] %(message)s"

_logging.addLevelName(TRACE, "TRACE")
_logger = _logging.getLogger("pulse_infer_amd")
_handler = None


class _Stderr(_logging.StreamHandler):
    """Writes to whatever ``sys.stderr`` is at the time of the message (a test may have replaced it)."""

    def __init__(self):
        super().__init__(sys.stderr)

    @property
    def stream(self):
        return sys.stderr

    @stream.setter
    def stream(self, value):
        pass


def _ready() -> _logging.Logger:
    global _handler
    if _handler is None:
        _handler = _Stderr()
        _handler.setFormatter(_logging.Formatter(DEFAULT_PATTERN))
        _logger.addHandler(_handler)
        _logger.propagate = False
        set_level(os.environ.get("PULSE_LOG_LEVEL", "info"))
    return _logger


def set_level(level) -> None:
    """A name (see the module's text) or a number of the standard ``logging`` module."""
    _ready() if _handler is None else None
    if isinstance(level, str):
        try:
            level = LEVELS[level.strip().lower()]
        except KeyError:
            raise ValueError(f"unknown log level '{level}'; choose from {', '.join(sorted(LEVELS))}") from None
    _logger.setLevel(int(level))


def set_pattern(pattern: str) -> None:
    """The format of a line, in the standard ``logging`` module's %-style (``%(levelname)s``, ``%(message)s``, ...)."""
    _ready()
    _handler.setFormatter(_logging.Formatter(pattern))


def enabled(level: str) -> bool:
    return _ready().isEnabledFor(LEVELS[level])


def trace(msg: str, *args) -> None:
    _ready().log(TRACE, msg, *args)


def debug(msg: str, *args) -> None:
    _ready().debug(msg, *args)


def info(msg: str, *args) -> None:
    _ready().info(msg, *args)


def warn(msg: str, *args) -> None:
    _ready().warning(msg, *args)


def error(msg: str, *args) -> None:
    _ready().error(msg, *args)


def fatal(msg: str, *args) -> None:
    _ready().critical(msg, *args)
