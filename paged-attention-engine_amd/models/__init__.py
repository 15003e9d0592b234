"""Architectures.  Importing this package registers every one of them."""
from . import danonex, qwen2, ritalorn  # noqa: F401
