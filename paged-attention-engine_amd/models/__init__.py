"""Architectures.  Importing this package registers every one of them."""
from . import dagavik, danonex, qwen2, ritalorn, zikezen  # noqa: F401
