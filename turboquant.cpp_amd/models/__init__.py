"""Architectures.  Importing this package registers every architecture it holds."""
from . import qwen2_moe  # noqa: F401
