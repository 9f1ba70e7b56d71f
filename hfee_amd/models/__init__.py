"""Architectures.  Importing this package registers every architecture it holds."""
from . import llama, ronavik, sabezen, vofezen  # noqa: F401
