from .compressed_attention import compressed_attention
from .linear_compress import linear_compress
from .topk_sparse_attention import topk_sparse_attention

__all__ = [
    "compressed_attention",
    "linear_compress",
    "topk_sparse_attention",
]
