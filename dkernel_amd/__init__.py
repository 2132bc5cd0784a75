"""MI355X-native block-sparse attention with the public API of `dkernel`
(reference: dkernel/__init__.py:1-12)."""
__version__ = "0.5.0"

from .interface import SparseAttention, LocalStrideSparseAttention, combine_attn_partitions
from .utils import get_sparse_attn_mask

__all__ = [
    "SparseAttention",
    "LocalStrideSparseAttention",
    "get_sparse_attn_mask",
    "combine_attn_partitions",
]
