"""Verbosity switch and ``(file:line): message`` debug printing (python/dtas/logging.py:6-19)."""
import inspect
import os

_LEVEL = 0


def set_log_level(level: int) -> None:
    global _LEVEL
    _LEVEL = int(level)


def get_log_level() -> int:
    return _LEVEL


def debug_info(msg) -> None:
    frame = inspect.currentframe().f_back
    print(f"({os.path.basename(frame.f_code.co_filename)}:{frame.f_lineno}): {msg}")
