"""Architectures.  Importing this package registers every one of them."""
from . import qwen2  # noqa: F401
