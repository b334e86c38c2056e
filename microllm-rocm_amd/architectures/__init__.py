"""Architectures this package provides; importing the package registers them."""
from . import gupitar, kalevik, qwen2, siditar, zabozen  # noqa: F401
