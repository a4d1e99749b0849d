"""Importing this package registers the architectures the library ships (GPT-2, Salopel, Kodatar)."""

from . import gpt2, kodatar, salopel  # noqa: F401
