"""Typed readers of config.json's values for configuration classes whose keys are nested objects: each names the
place of the offending key in its error."""
from __future__ import annotations

from .errors import ConfigError


def obj(d, key, where):
    v = d.get(key) if isinstance(d, dict) else None
    if not isinstance(v, dict):
        raise ConfigError(f"{where}: {key!r} must be an object")
    return v


def integer(d, key, where, least=1):
    v = d.get(key)
    if isinstance(v, bool) or not isinstance(v, (int, float)) or int(v) != v:
        raise ConfigError(f"{where}: {key!r} must be an integer, got {v!r}")
    if int(v) < least:
        raise ConfigError(f"{where}: {key!r} == {v} (must be at least {least})")
    return int(v)


def number(d, key, where):
    v = d.get(key)
    if isinstance(v, bool) or not isinstance(v, (int, float)):
        raise ConfigError(f"{where}: {key!r} must be a number, got {v!r}")
    return float(v)
