"""Architectures.  Importing this package registers every architecture it holds."""
from . import llama, vofezen  # noqa: F401
