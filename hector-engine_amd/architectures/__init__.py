"""Architectures known to the registry."""
from . import qwen2, volonex  # noqa: F401
