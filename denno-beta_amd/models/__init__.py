"""Architectures the framework ships.  Importing a module registers it."""
from . import dogalorn, gpt2, nigilorn, pafivik, ridopel   # noqa: F401
