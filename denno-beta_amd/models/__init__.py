"""Architectures the framework ships.  Importing a module registers it."""
from . import gpt2   # noqa: F401
