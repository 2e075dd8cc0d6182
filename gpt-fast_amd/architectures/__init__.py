"""Architectures this library knows.  Importing a module registers its architecture."""
from . import llama, nizedra, pigodra, vusenex  # noqa: F401
