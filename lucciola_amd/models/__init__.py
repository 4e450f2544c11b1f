"""Architectures: importing this package registers them."""
from . import kikunex, larupel, pubodra, qwen3, rununex  # noqa: F401
