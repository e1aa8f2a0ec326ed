"""Architectures.  Importing the package registers them."""
from . import llama, mifidra, vafodra, vupelorn  # noqa: F401
