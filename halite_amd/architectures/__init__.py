"""Architectures: each module registers itself in ``config.registry`` on import."""

from . import kavuvik, llama, vepitar, zabunex  # noqa: F401
