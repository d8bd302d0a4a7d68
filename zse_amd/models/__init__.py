"""Importing this package registers every architecture the engine serves."""
from . import gemma2  # noqa: F401
