"""Architectures. Importing this package registers them."""
from . import qwen2, goridra, tobozen, mobupel   # noqa: F401
