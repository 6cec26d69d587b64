"""Reading typed values out of a ``config.json`` dictionary.

An architecture's configuration class names the keys it reads, their types and
defaults; every problem found while reading (missing key, wrong type, a value
the architecture does not support) is collected and raised as one
``ConfigError`` that lists all of them, in the manner of the reference's
pinned-config check (engine/dryft_qwen3/config.py:121-135).
"""

from __future__ import annotations

import json
import os
from typing import Any, Callable

_MISSING = object()


class ConfigError(ValueError):
    """One error for a whole config.json: ``problems`` holds every finding."""

    def __init__(self, what: str, problems: list[str]):
        self.problems = list(problems)
        super().__init__(what + ":\n  " + "\n  ".join(self.problems))


class KeyReader:
    """Pulls keys out of a raw config dictionary and remembers what went wrong."""

    def __init__(self, raw: dict[str, Any]):
        if not isinstance(raw, dict):
            raise ConfigError("config.json", ["top level is not a JSON object"])
        self.raw = raw
        self.problems: list[str] = []

    def _get(self, key: str, default: Any) -> Any:
        if key in self.raw and self.raw[key] is not None:
            return self.raw[key]
        if default is _MISSING:
            self.problems.append(f"{key}: missing")
            return None
        return default

    def integer(self, key: str, default: Any = _MISSING, minimum: int = 1) -> int:
        v = self._get(key, default)
        if v is None:
            return 0
        if isinstance(v, bool) or not isinstance(v, int):
            if isinstance(v, float) and v == int(v):
                v = int(v)
            else:
                self.problems.append(f"{key}: expected an integer, got {v!r}")
                return 0
        if v < minimum:
            self.problems.append(f"{key}: must be >= {minimum}, got {v}")
        return int(v)

    def number(self, key: str, default: Any = _MISSING, positive: bool = True) -> float:
        v = self._get(key, default)
        if v is None:
            return 0.0
        if isinstance(v, bool) or not isinstance(v, (int, float)):
            self.problems.append(f"{key}: expected a number, got {v!r}")
            return 0.0
        if positive and not v > 0:
            self.problems.append(f"{key}: must be > 0, got {v}")
        return float(v)

    def boolean(self, key: str, default: Any = _MISSING) -> bool:
        v = self._get(key, default)
        if v is None:
            return False
        if not isinstance(v, bool):
            self.problems.append(f"{key}: expected true/false, got {v!r}")
            return False
        return v

    def require(self, key: str, ok: Callable[[Any], bool], default: Any, why: str) -> None:
        """A key that is only validated: its value must satisfy ``ok``."""
        v = self.raw.get(key, default)
        if not ok(v):
            self.problems.append(f"{key}: {why}, got {v!r}")

    def check(self, condition: bool, message: str) -> None:
        if not condition:
            self.problems.append(message)

    def finish(self, what: str) -> None:
        if self.problems:
            raise ConfigError(what, self.problems)


def read_config_json(model_dir: str) -> dict[str, Any]:
    path = os.path.join(model_dir, "config.json")
    if not os.path.isfile(path):
        raise FileNotFoundError(f"no config.json in {model_dir}")
    with open(path, "r", encoding="utf-8") as f:
        return json.load(f)
