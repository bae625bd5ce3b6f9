"""Architectures: importing this package registers them."""
from . import pubodra, qwen3  # noqa: F401
