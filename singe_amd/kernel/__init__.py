"""Counterpart of the ``singe-kernel`` crate's CUDA surface for the attention path."""
from . import attention  # noqa: F401
