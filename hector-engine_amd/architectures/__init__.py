"""Architectures known to the registry."""
from . import butolorn, penasun, qwen2, volonex  # noqa: F401
