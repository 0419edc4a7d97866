"""Compressed attention + top-k block selection under the reference's names
(nsa_ref/ops/compressed_attention.py:762-829 autograd Function, :1161-1317 entry point)."""
from __future__ import annotations

import math
import warnings
from typing import Tuple, Union

import torch

from fsa_hip import ops as _ops


class CompressedAttention(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q, k, v, kernel_size, kernel_stride, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k,
                sm_scale=None):
        assert q.dtype == torch.bfloat16 or q.dtype == torch.float16
        assert q.dtype == k.dtype and k.dtype == v.dtype
        assert cu_seqlens_q.dtype == torch.int32 and cu_seqlens_k.dtype == torch.int32
        if sm_scale is None:
            sm_scale = 1 / math.sqrt(q.shape[-1])
        o, lse = _ops.cmpattn_fwd(q, k, v, kernel_size, kernel_stride, cu_seqlens_q, cu_seqlens_k, max_seqlen_q,
                                  sm_scale)
        ctx.save_for_backward(q, k, v, o, lse, cu_seqlens_q, cu_seqlens_k)
        ctx.sm_scale = sm_scale
        ctx.max_seqlen_q = max_seqlen_q
        ctx.kernel_size = kernel_size
        ctx.kernel_stride = kernel_stride
        return o, lse

    @staticmethod
    def backward(ctx, do, *args):
        q, k, v, o, lse, cu_q, cu_k = ctx.saved_tensors
        dq, dk, dv = _ops.cmpattn_bwd(q, k, v, o, do, lse, ctx.kernel_size, ctx.kernel_stride, cu_q, cu_k,
                                      ctx.max_seqlen_q, ctx.sm_scale)
        return dq, dk, dv, None, None, None, None, None, None, None


def compressed_attention(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    kernel_size: int,
    kernel_stride: int,
    block_size: int,
    topk: int,
    cu_seqlens_q: torch.Tensor,
    cu_seqlens_k: torch.Tensor,
    max_seqlen_q: int,
    max_seqlen_k: int,
    sm_scale: float = None,
    init_blocks: int = 1,
    local_blocks: int = 2,
    parallel_topk_compute: Union[str, bool] = False,
    score_head_as_written: bool = False,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Attention between the queries and the compressed keys / values, and the top-k block ids
    [num_kv_heads, total_q, min(topk, ceil(max_seqlen_q / block_size))] used by the selected attention.

    `parallel_topk_compute` decides whether the block scores are rounded to bf16 before the selection
    (False, the reference's per-head path, the only one its callers use) or kept in fp32 (True).  The
    reference's parallel path also hands the unsliced q to its score kernel, which then scores kv head
    kh with q head kh instead of the first head of group kh (nsa_ref/ops/compressed_attention.py:870,
    898, 906 against :1280-1283); `score_head_as_written=True` together with
    `parallel_topk_compute=True` reproduces that literally, the default scores every kv head with the
    first q head of its group on both paths."""
    if max_seqlen_q is None:
        max_seqlen_q = (cu_seqlens_q[1:] - cu_seqlens_q[:-1]).max().item()
    if max_seqlen_k is None:
        max_seqlen_k = (cu_seqlens_k[1:] - cu_seqlens_k[:-1]).max().item()
    if sm_scale is None:
        sm_scale = 1 / math.sqrt(q.shape[-1])
    attn_output, lse = CompressedAttention.apply(q, k, v, kernel_size, kernel_stride, cu_seqlens_q, cu_seqlens_k,
                                                 max_seqlen_q, max_seqlen_k, sm_scale)
    if topk <= 0:
        warnings.warn("topk <= 0, returned topk_idx will be None")
        return attn_output, None
    assert topk >= init_blocks + local_blocks
    if parallel_topk_compute == "auto":
        parallel_topk_compute = q.shape[0] <= 32768
    with torch.no_grad():
        topk_idx = _ops.cmp_topk(q, k, lse, kernel_size, kernel_stride, block_size, topk, cu_seqlens_q, cu_seqlens_k,
                                 max_seqlen_q, max_seqlen_k, init_blocks, local_blocks, sm_scale,
                                 scores_to_bf16=not parallel_topk_compute,
                                 score_head_as_written=bool(score_head_as_written and parallel_topk_compute))
    return attn_output, topk_idx
