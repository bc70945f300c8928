"""Python surface of sparse-mask attention for MI355X; same exports as the reference's python/__init__.py:1-3."""
from .sparse_attention import sparse_attention, sparse_attention_func  # noqa: F401

__all__ = ["sparse_attention", "sparse_attention_func"]
