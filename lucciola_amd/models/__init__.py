"""Architectures: importing this package registers them."""
from . import larupel, pubodra, qwen3  # noqa: F401
