"""Architectures this package provides; importing the package registers them."""
from . import qwen2  # noqa: F401
