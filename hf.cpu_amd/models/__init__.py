"""Architectures. Importing this package registers them."""
from . import qwen2, goridra   # noqa: F401
