"""Architectures.  Importing this package registers every architecture it holds."""
from . import felepel, qwen2_moe, taminex  # noqa: F401
