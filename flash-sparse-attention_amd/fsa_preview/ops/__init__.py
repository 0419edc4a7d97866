from .compressed_attention_decode import _compressed_attention_decode
from .linear_compress_decode import _linear_compress_decode
from .selected_attention_decode import _topk_sparse_attention_decode

__all__ = [
    "_linear_compress_decode",
    "_compressed_attention_decode",
    "_topk_sparse_attention_decode",
]
