from .fsa_decode import FlashSparseAttentionDecode
from .fsa_decode_kernel import FlashSparseAttentionDecodeKernel

__all__ = ["FlashSparseAttentionDecode", "FlashSparseAttentionDecodeKernel"]
