"""Architectures this package provides; importing the package registers them."""
from . import gupitar, qwen2, siditar, zabozen  # noqa: F401
