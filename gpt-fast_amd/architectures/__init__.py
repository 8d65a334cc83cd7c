"""Architectures this library knows.  Importing a module registers its architecture."""
from . import llama, pigodra  # noqa: F401
