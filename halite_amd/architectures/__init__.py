"""Architectures: each module registers itself in ``config.registry`` on import."""

from . import diporax, kavuvik, llama, vepitar, zabunex  # noqa: F401
