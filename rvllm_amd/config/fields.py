"""Strict readers for config.json fields.

Every reader records a problem instead of raising, so that the caller can
report all of them at once.  The reference's readers are strict in the same
way: a key of the wrong JSON type is "missing or invalid", never coerced
(v3/crates/rvllm-loader/src/gemma4_arch.rs:138-153,
v3/crates/rvllm-core/src/config/hf.rs:9-119).
"""

from __future__ import annotations

import math
from typing import Any, Iterable, Optional

_MISSING = object()


class FieldReader:
    """Reads typed fields out of one JSON object and remembers what went wrong."""

    def __init__(self, obj: dict, outer: Optional[dict] = None):
        self.obj = obj
        self.outer = outer if outer is not None else {}
        self.problems: list[str] = []
        self.used: set[str] = set()

    def _lookup(self, keys: Iterable[str]) -> tuple[str, Any]:
        keys = list(keys)
        for key in keys:
            if key in self.obj and self.obj[key] is not None:
                self.used.add(key)
                return key, self.obj[key]
        for key in keys:
            if key in self.outer and self.outer[key] is not None:
                return key, self.outer[key]
        return keys[0], _MISSING

    def has(self, *keys: str) -> bool:
        return self._lookup(keys)[1] is not _MISSING

    def integer(self, *keys: str, default: Any = _MISSING, lo: int = 0, hi: int = 1 << 62) -> int:
        key, value = self._lookup(keys)
        if value is _MISSING:
            if default is not _MISSING:
                return default
            self.problems.append(f"missing or invalid required field {keys[0]}")
            return lo
        if isinstance(value, bool) or not isinstance(value, int):
            self.problems.append(f"field {key} must be an integer, got {value!r}")
            return lo
        if not (lo <= value <= hi):
            self.problems.append(f"field {key}={value} must be in {lo}..={hi}")
            return lo
        return value

    def real(self, *keys: str, default: Any = _MISSING, positive: bool = False) -> float:
        key, value = self._lookup(keys)
        if value is _MISSING:
            if default is not _MISSING:
                return default
            self.problems.append(f"missing or invalid required field {keys[0]}")
            return 1.0
        if isinstance(value, bool) or not isinstance(value, (int, float)):
            self.problems.append(f"field {key} must be a number, got {value!r}")
            return 1.0
        value = float(value)
        if not math.isfinite(value):
            self.problems.append(f"field {key} must be finite")
            return 1.0
        if positive and not value > 0.0:
            self.problems.append(f"field {key}={value} must be > 0")
            return 1.0
        return value

    def boolean(self, *keys: str, default: Any = _MISSING) -> bool:
        key, value = self._lookup(keys)
        if value is _MISSING:
            if default is not _MISSING:
                return default
            self.problems.append(f"missing or invalid required field {keys[0]}")
            return False
        if not isinstance(value, bool):
            self.problems.append(f"field {key} must be a boolean, got {value!r}")
            return False
        return value

    def string(self, *keys: str, default: Any = _MISSING) -> str:
        key, value = self._lookup(keys)
        if value is _MISSING:
            if default is not _MISSING:
                return default
            self.problems.append(f"missing or invalid required field {keys[0]}")
            return ""
        if not isinstance(value, str):
            self.problems.append(f"field {key} must be a string, got {value!r}")
            return ""
        return value

    def raw(self, *keys: str) -> Any:
        value = self._lookup(keys)[1]
        return None if value is _MISSING else value

    def problem(self, text: str) -> None:
        self.problems.append(text)
