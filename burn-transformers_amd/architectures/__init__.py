"""Importing this package registers the architectures the library ships (GPT-2, Salopel, Kodatar, Rotutar)."""

from . import gpt2, kodatar, rotutar, salopel  # noqa: F401
