"""Importing this package registers every architecture the engine serves."""
from . import dafotar, gemma2  # noqa: F401
