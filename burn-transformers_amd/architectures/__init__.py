"""Importing this package registers the architectures the library ships (GPT-2)."""

from . import gpt2  # noqa: F401
