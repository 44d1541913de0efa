"""Architectures.  Importing the package registers them."""
from . import llama, vafodra, vupelorn  # noqa: F401
