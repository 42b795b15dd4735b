"""Architectures known to the engine.  Importing this package registers them."""
from . import llama  # noqa: F401
