"""Mirrors ``src/cuda_extension/co_me/__init__.py``: exposes the ``co_me_cuext`` module."""

from . import co_me_cuext  # noqa: F401
