"""Architectures known to the framework; importing this package registers them."""
from . import qwen2  # noqa: F401
