"""Architectures known to the registry.  Importing the package registers them."""
from . import qwen2  # noqa: F401
