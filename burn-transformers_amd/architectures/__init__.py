"""Importing this package registers the architectures the library ships (GPT-2, Salopel)."""

from . import gpt2, salopel  # noqa: F401
