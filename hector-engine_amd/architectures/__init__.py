"""Architectures known to the registry."""
from . import penasun, qwen2, volonex  # noqa: F401
