"""Opt-in call counters keyed "<OpClass>-<backend>" (xma/counters.py:10-44)."""

from __future__ import annotations

from collections import Counter
from contextlib import contextmanager
from typing import Any, Iterator


_counts: Counter = Counter()
_enabled = False


def is_counter_enabled() -> bool:
    return _enabled


@contextmanager
def enable_counters() -> Iterator[None]:
    global _enabled
    _enabled = True
    try:
        yield
    finally:
        _enabled = False


def increment_counter(key: Any, value: int = 1) -> None:
    if _enabled:
        _counts[key] += value


def reset_counters() -> None:
    _counts.clear()


def get_counter_value(key: Any) -> int:
    return _counts[key]
