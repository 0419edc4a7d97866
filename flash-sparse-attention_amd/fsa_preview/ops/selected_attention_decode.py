"""One-step decode of the selected branch under the reference's name
(fsa_preview/ops/selected_attention_decode.py:8-42).

The reference calls its prefill kernel with a query of length one, which keeps key 0 only
(nsa_ref/ops/topk_sparse_attention.py:116-119,162); `as_written=True` reproduces that, the default
attends every cached key of the selected blocks."""
import math

import torch

from fsa_hip import ops as _ops


def _topk_sparse_attention_decode(
    q: torch.Tensor,  # [1, num_q_heads, head_dim]
    k: torch.Tensor,  # [cache_len, num_kv_heads, head_dim] (new token appended)
    v: torch.Tensor,
    topk_idx: torch.Tensor,  # [num_kv_heads, 1, topk]
    block_size: int,
    cu_seqlens_q: torch.Tensor,
    cu_seqlens_k: torch.Tensor,
    max_seqlen_q=None,
    max_seqlen_k=None,
    sm_scale=None,
    as_written: bool = False,
):
    assert q.dtype == torch.bfloat16 or q.dtype == torch.float16
    assert q.dtype == k.dtype and k.dtype == v.dtype
    assert topk_idx.dtype == torch.int32
    assert cu_seqlens_q.dtype == torch.int32 and cu_seqlens_k.dtype == torch.int32
    if sm_scale is None:
        sm_scale = 1 / math.sqrt(q.shape[-1])
    if as_written:
        cu1 = torch.tensor([0, 1], dtype=torch.int32, device=q.device)
        only0 = torch.zeros((k.shape[1], 1, 1), dtype=torch.int32, device=q.device)
        o, _ = _ops.decode_selattn(q, k[:1], v[:1], cu1, only0, block_size, sm_scale)
        return o
    o, _ = _ops.decode_selattn(q, k, v, cu_seqlens_k, topk_idx.contiguous(), block_size, sm_scale)
    return o
