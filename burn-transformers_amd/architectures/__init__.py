"""Importing this package registers the architectures the library ships (GPT-2, Salopel, Kodatar, Rotutar, Gavasun)."""

from . import gavasun, gpt2, kodatar, rotutar, salopel  # noqa: F401
