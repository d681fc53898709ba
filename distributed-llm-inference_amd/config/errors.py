"""Errors raised while reading a model's ``config.json``."""

from __future__ import annotations


class ConfigError(ValueError):
    """The configuration cannot be used."""


class UnsupportedModelError(ConfigError):
    """The checkpoint asks for an architecture feature that the engine does not implement.

    Refusing is deliberate: a feature that is silently ignored (a sliding window, an unknown
    rotary variant) gives fluent but wrong text (reference: src/dli/model/config.py:3-6).
    """


class MissingConfigKeyError(KeyError, ConfigError):
    """A key that has no default is absent from ``config.json``."""

    def __init__(self, key: str) -> None:
        super().__init__(key)
        self.key = key

    def __str__(self) -> str:
        return f"config.json has no {self.key!r} and the architecture gives it no default"
