"""Logging / assertion helpers with the reference's names and error behaviour.

Mirrors ``pace/utils/logging.py:63-150`` of the reference: ``PACE_ASSERT`` logs
and raises ``AssertionError(message)``; the ``PACE_LLM_*`` variants tag the line
with ``-llm``.  The threshold comes from ``PACE_LOG_LEVEL``
(``csrc/core/logging.h:69-132``).
"""
from __future__ import annotations

import os
import sys
from typing import Optional

_LEVELS = {"debug": 0, "profile": 1, "info": 2, "warning": 3, "error": 4, "none": 5}


def _threshold() -> int:
    return _LEVELS.get(os.getenv("PACE_LOG_LEVEL", "warning").lower(), 3)


def _emit(level: str, message: str, extra_info: Optional[str]) -> None:
    if _LEVELS[level] >= _threshold():
        sys.stdout.write(f"[{level.upper()}] pace{extra_info or ''}: {message}\n")


def PACE_DEBUG(message: str, extra_info: Optional[str] = None, caller_stack_depth: int = 1) -> None:
    _emit("debug", message, extra_info)


def PACE_INFO(message: str, extra_info: Optional[str] = None, caller_stack_depth: int = 1) -> None:
    _emit("info", message, extra_info)


def PACE_WARNING(message: str, extra_info: Optional[str] = None, caller_stack_depth: int = 1) -> None:
    _emit("warning", message, extra_info)


def PACE_ASSERT(condition: bool, message: str, extra_info: Optional[str] = None, caller_stack_depth: int = 1) -> None:
    if not condition:
        _emit("error", message, extra_info)
        raise AssertionError(message)


def PACE_LLM_DEBUG(message: str, caller_stack_depth: int = 2) -> None:
    PACE_DEBUG(message, extra_info="-llm ")


def PACE_LLM_ASSERT(condition: bool, message: str, caller_stack_depth: int = 2) -> None:
    PACE_ASSERT(condition, message, extra_info="-llm ")
