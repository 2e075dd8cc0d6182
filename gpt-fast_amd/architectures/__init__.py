"""Architectures this library knows.  Importing a module registers its architecture."""
from . import llama, nizedra, pigodra, refolix, vusenex  # noqa: F401
