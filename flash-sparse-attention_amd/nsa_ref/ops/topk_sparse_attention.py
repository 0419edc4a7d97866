"""The NSA-named selected-attention surface of the reference
(nsa_ref/ops/topk_sparse_attention.py): `_topk_sparse_attention_fwd` (:814-905),
`_topk_sparse_attention_bwd` (:908-1100), `TopkSparseAttention` (:1102-1172),
`topk_sparse_attention` (:1174-1210) and `reorder_topk_idx` (:412-476), with the
reference's argument order, asserts and return values.

The reference keeps two implementations of the same operator - this query-major
one and the block-major FSA one - and its own test compares them
(test/test_FSA_optimized_sel_attn.py:142-237).  Here both sets of names run the
same gfx950 kernels behind the C ABI: the kernels gather (query, head) rows, so
one implementation serves every GQA group size.  `backward_sum_o_do` (:197-230)
is a Triton kernel object launched with grid syntax, not a Python function; its
role is the delta kernel inside `fsa_selattn_bwd`.
"""
from __future__ import annotations

import math
from typing import Any, Optional

import torch

from fsa.ops.FSA_topk_sparse_attention import _BLOCK_SIZES, _build_kernel_index
from fsa_hip import ops as _ops


def _topk_sparse_attention_fwd(
    q: torch.Tensor,  # [total_len, num_q_heads, head_dim]
    k: torch.Tensor,  # [total_len, num_k_heads, head_dim]
    v: torch.Tensor,  # [total_len, num_k_heads, head_dim]
    topk_idx: torch.Tensor,  # [num_kv_heads, total_len, topk]
    block_size: int,
    cu_seqlens_q: torch.Tensor,
    cu_seqlens_k: torch.Tensor,
    max_seqlen_q: int,
    max_seqlen_k: int,
    sm_scale: float,
):
    """(o, lse): lse is [num_q_heads, total_len] fp32, base 2."""
    assert k.dtype == q.dtype and v.dtype == q.dtype
    assert cu_seqlens_q.dtype == torch.int32 and cu_seqlens_k.dtype == torch.int32
    assert block_size in _BLOCK_SIZES
    assert q.shape[1] % k.shape[1] == 0
    index, _ = _build_kernel_index(topk_idx, cu_seqlens_q, block_size)
    return _ops.selattn_fwd(q, k, v, index, sm_scale)


def _topk_sparse_attention_bwd(
    o: torch.Tensor,
    do: torch.Tensor,
    lse: torch.Tensor,
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    topk_idx: torch.Tensor,
    block_size: int,
    cu_seqlens_q: torch.Tensor,
    cu_seqlens_k: torch.Tensor,
    max_seqlen_q: int,
    max_seqlen_k: int,
    sm_scale: float,
):
    """(dq, dk, dv); dk / dv are already summed over the query heads of a group."""
    assert block_size in _BLOCK_SIZES
    index, _ = _build_kernel_index(topk_idx, cu_seqlens_q, block_size)
    return _ops.selattn_bwd(q, k, v, o, do, lse, index, sm_scale)


class TopkSparseAttention(torch.autograd.Function):
    @staticmethod
    def forward(
        ctx,
        q: torch.Tensor,
        k: torch.Tensor,
        v: torch.Tensor,
        topk_idx: torch.Tensor,
        block_size: int,
        cu_seqlens_q: torch.Tensor,
        cu_seqlens_k: torch.Tensor,
        max_seqlen_q,
        max_seqlen_k,
        sm_scale=None,
    ):
        assert q.dtype == torch.bfloat16 or q.dtype == torch.float16
        assert q.dtype == k.dtype and k.dtype == v.dtype
        assert topk_idx.dtype == torch.int32
        assert cu_seqlens_q.dtype == torch.int32 and cu_seqlens_k.dtype == torch.int32
        if sm_scale is None:
            sm_scale = 1 / math.sqrt(q.shape[-1])
        o, lse = _topk_sparse_attention_fwd(q, k, v, topk_idx, block_size, cu_seqlens_q, cu_seqlens_k,
                                            max_seqlen_q, max_seqlen_k, sm_scale)
        ctx.save_for_backward(q, k, v, o, lse, cu_seqlens_q, cu_seqlens_k, topk_idx)
        ctx.sm_scale = sm_scale
        ctx.max_seqlen_q = max_seqlen_q
        ctx.max_seqlen_k = max_seqlen_k
        ctx.block_size = block_size
        return o

    @staticmethod
    def backward(ctx, do: torch.Tensor, *args) -> Any:
        q, k, v, o, lse, cu_seqlens_q, cu_seqlens_k, topk_idx = ctx.saved_tensors
        assert ctx.block_size in _BLOCK_SIZES
        dq, dk, dv = _topk_sparse_attention_bwd(o, do, lse, q, k, v, topk_idx, ctx.block_size, cu_seqlens_q,
                                                cu_seqlens_k, ctx.max_seqlen_q, ctx.max_seqlen_k, ctx.sm_scale)
        return dq, dk, dv, None, None, None, None, None, None, None, None


def topk_sparse_attention(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    topk_idx: torch.Tensor,
    block_size: int,
    cu_seqlens: torch.Tensor,
    softmax_scale: Optional[float] = None,
) -> torch.Tensor:
    """Top-k sparse attention, varlen: [total_len, num_q_heads, head_dim] out; -1 in topk_idx is padding."""
    # per-sequence sizes are derived on the device: no host read of max_seqlen as in the reference (:1197)
    return TopkSparseAttention.apply(q, k, v, topk_idx, block_size, cu_seqlens, cu_seqlens, None, None,
                                     softmax_scale)


def reorder_topk_idx(
    topk_idx: torch.Tensor,
    cu_topk_q_count: torch.Tensor,
    cu_seqlens: torch.Tensor,
    cu_seqblocks: torch.Tensor,
    block_size: int,
):
    """topk_q_idx [num_kv_heads, max_h cu_topk_q_count[h, -1]] int32: for every kv block (all sequences
    numbered through, cu_seqblocks) the sequence-local ids of the queries that selected it, -1 behind the
    last one.  The reference orders the ids of a block by an unstable argsort; here they ascend."""
    assert block_size in _BLOCK_SIZES
    index = _ops.build_index(topk_idx, cu_seqlens, block_size)
    width = int(cu_topk_q_count[:, -1].max().item())
    tok = index.sel_tokens[:, :width].to(torch.int64)
    seq = torch.searchsorted(cu_seqlens.to(torch.int64), tok.clamp(min=0), right=True) - 1
    local = tok - cu_seqlens.to(torch.int64)[seq]
    return torch.where(tok >= 0, local, torch.full_like(local, -1)).to(torch.int32)
