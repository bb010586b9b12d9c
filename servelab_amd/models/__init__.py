"""Importing this package registers the architectures it holds."""
from . import qwen2  # noqa: F401
