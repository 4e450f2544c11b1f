"""Architectures: importing this package registers them."""
from . import kikunex, larupel, pubodra, qwen3  # noqa: F401
