"""Architectures known to the registry."""
from . import butolorn, domorax, penasun, qwen2, volonex  # noqa: F401
