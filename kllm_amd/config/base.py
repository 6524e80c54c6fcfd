"""Typed configuration: the shared machinery.

A configuration class declares which ``config.json`` keys it reads, their
defaults and what it refuses.  Nothing that ``config.json`` gives is written
down anywhere else in the package.
"""

from __future__ import annotations

import json
import os
from dataclasses import dataclass, fields, asdict


class ConfigError(ValueError):
    """A config.json that cannot be run as asked: a key is missing, has a bad
    value, or names an option this engine does not implement."""


_MISSING = object()


class KeyReader:
    """Reads keys of a config.json dict and remembers which were used, so that
    problems can be reported with the key's name."""

    def __init__(self, raw: dict, where: str = "config.json"):
        if not isinstance(raw, dict):
            raise ConfigError(f"{where}: expected a JSON object, got {type(raw).__name__}")
        self.raw = raw
        self.where = where

    def has(self, key):
        return key in self.raw and self.raw[key] is not None

    def get(self, key, default=_MISSING):
        if self.has(key):
            return self.raw[key]
        if default is _MISSING:
            raise ConfigError(f"{self.where}: required key '{key}' is missing")
        return default

    def positive_int(self, key, default=_MISSING):
        v = self.get(key, default)
        if v is None:
            return None
        if isinstance(v, bool) or not isinstance(v, int) or v <= 0:
            raise ConfigError(f"{self.where}: '{key}' must be a positive integer, got {v!r}")
        return v

    def positive_float(self, key, default=_MISSING):
        v = self.get(key, default)
        if isinstance(v, bool) or not isinstance(v, (int, float)) or not v > 0:
            raise ConfigError(f"{self.where}: '{key}' must be a positive number, got {v!r}")
        return float(v)

    def boolean(self, key, default=_MISSING):
        v = self.get(key, default)
        if not isinstance(v, bool):
            raise ConfigError(f"{self.where}: '{key}' must be true or false, got {v!r}")
        return v

    def refuse_unless(self, key, allowed, why):
        """The key may be absent, null, or one of ``allowed``."""
        if self.has(key) and self.raw[key] not in allowed:
            raise ConfigError(f"{self.where}: '{key}' = {self.raw[key]!r} is not supported ({why})")


@dataclass(frozen=True)
class ModelConfig:
    """Base of every architecture's typed configuration."""

    architecture: str

    def to_dict(self) -> dict:
        """The config.json form of this configuration."""
        raise NotImplementedError

    def describe(self) -> dict:
        return asdict(self)

    def field_names(self):
        return [f.name for f in fields(self)]


def read_config_json(model_dir: str) -> dict:
    path = os.path.join(model_dir, "config.json")
    try:
        with open(path, "r", encoding="utf-8") as f:
            return json.load(f)
    except FileNotFoundError:
        raise ConfigError(f"{path}: no such file") from None
    except json.JSONDecodeError as e:
        raise ConfigError(f"{path}: not valid JSON ({e})") from None
