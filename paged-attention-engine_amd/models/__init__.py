"""Architectures.  Importing this package registers every one of them."""
from . import danonex, qwen2  # noqa: F401
