"""Architectures. Importing this package registers them."""
from . import qwen2, goridra, tobozen, mobupel, gitasun   # noqa: F401
