"""Architectures.  Importing this package registers every architecture it holds."""
from . import llama, ronavik, sabezen, saposun, vofezen  # noqa: F401
