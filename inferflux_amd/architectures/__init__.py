"""Architectures known to the registry.  Importing the package registers them."""
from . import mumusun, podurax, qwen2, tabatar, vavadra  # noqa: F401
