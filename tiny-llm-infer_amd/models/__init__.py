"""Architectures this engine knows.  Importing the package registers them."""
from . import qwen3  # noqa: F401
