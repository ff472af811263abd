"""Operator package with the reference's public surface (``self_ops/__init__.py:1`` re-exports ``ops_py``)."""
from .ops_py import *  # noqa: F401,F403
from .ops_py import __all__  # noqa: F401
