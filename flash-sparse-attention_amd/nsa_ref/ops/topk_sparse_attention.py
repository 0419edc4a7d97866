"""`topk_sparse_attention` under the reference's name (nsa_ref/ops/topk_sparse_attention.py:1174-1210).

The reference keeps a second, query-major kernel for GQA groups above 8; the gfx950
kernels gather (query, head) rows, so one implementation serves every group size."""
from typing import Optional

import torch

from fsa.ops.FSA_topk_sparse_attention import FSA_topk_sparse_attention


def topk_sparse_attention(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    topk_idx: torch.Tensor,
    block_size: int,
    cu_seqlens: torch.Tensor,
    softmax_scale: Optional[float] = None,
) -> torch.Tensor:
    return FSA_topk_sparse_attention(q, k, v, topk_idx, block_size, cu_seqlens, softmax_scale)
