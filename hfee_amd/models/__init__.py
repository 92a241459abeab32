"""Architectures.  Importing this package registers every architecture it holds."""
from . import llama, sabezen, vofezen  # noqa: F401
