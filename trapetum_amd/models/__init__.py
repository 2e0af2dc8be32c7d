"""Architectures; importing this package registers the built-in ones."""
from . import gemma2   # noqa: F401
