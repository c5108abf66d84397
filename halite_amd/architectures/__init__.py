"""Architectures: each module registers itself in ``config.registry`` on import."""

from . import llama  # noqa: F401
