"""Architectures. Importing this package registers them."""
from . import qwen2, goridra, tobozen   # noqa: F401
