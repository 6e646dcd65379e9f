"""Architectures known to the registry.  Importing the package registers them."""
from . import mumusun, podurax, qwen2, tabatar  # noqa: F401
