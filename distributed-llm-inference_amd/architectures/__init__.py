"""Architectures that ship with the engine. Importing this package registers them."""

from . import llama  # noqa: F401
