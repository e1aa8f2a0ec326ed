"""Architectures.  Importing the package registers them."""
from . import llama, mifidra, sofinex, vafodra, vupelorn  # noqa: F401
