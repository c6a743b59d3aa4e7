"""Architectures this library knows.  Importing a module registers its architecture."""
from . import llama  # noqa: F401
