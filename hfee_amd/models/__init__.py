"""Architectures.  Importing this package registers every architecture it holds."""
from . import llama  # noqa: F401
