"""Architectures.  Importing this package registers every architecture it holds."""
from . import beronex, bosalix, felepel, qwen2_moe, taminex  # noqa: F401
