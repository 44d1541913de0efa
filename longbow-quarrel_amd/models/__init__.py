"""Architectures.  Importing the package registers them."""
from . import llama, vafodra  # noqa: F401
