"""Architectures.  Importing this package registers every one of them."""
from . import dagavik, danonex, qwen2, ritalorn  # noqa: F401
