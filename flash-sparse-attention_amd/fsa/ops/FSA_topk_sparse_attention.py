"""Selected (top-k block sparse) attention under the reference's names.

Mirrors the public surface of fsa/ops/FSA_topk_sparse_attention.py of the
reference (functional forms :569-618 and :1715-1884, autograd Function
:1887-1961, user entry point :1964-2000): same argument order, dtypes, asserts
and return values.  All computation happens in the gfx950 kernels behind the C
ABI; nothing here falls back to PyTorch math.
"""
from __future__ import annotations

import math
from typing import Any, Optional

import torch

from fsa_hip import ops as _ops

_BLOCK_SIZES = {32, 64, 128, 256}


class PermuteResults(list):
    """What the forward hands to the backward: the inverted block->query index.

    The reference returns one dict per sequence (FSA_topk_sparse_attention.py:
    990-997, 1024-1026).  Indexing this object builds those dicts on demand from
    the device-resident CSR index (a host copy of cu_seqlens is needed, so it
    synchronises); the backward only uses `.index`.
    """

    def __init__(self, index: _ops.SelIndex, ref_args=None):
        super().__init__()
        self.index = index          # what the kernels use
        self._ref_args = ref_args   # (topk_idx, cu_seqlens, block_size) when the caller's block size differs
        self._built = False

    def _build(self):
        if self._built:
            return
        ix = self.index if self._ref_args is None else _ops.build_index(*self._ref_args)
        cu = ix.cu_seqlens.cpu().tolist()
        cub = ix.cu_blocks.cpu().tolist()
        for s in range(ix.batch):
            real_nb = cub[s + 1] - cub[s]
            nb = max(real_nb, ix.topk)
            lens_all = torch.zeros((ix.num_kv_heads, nb), dtype=torch.int32, device=ix.counts.device)
            lens_all[:, :real_nb] = ix.counts[:, cub[s]:cub[s + 1]]
            d = {
                "global_max_valid_tokens": lens_all[:, 1:].max() if nb > 1 else lens_all.max(),
                "num_blocks": nb,
                "real_num_blocks": real_nb,
                "valid_lens_all": lens_all,
                "valid_topk_idx_permuted_tile": [],
                "valid_lens": [],
                "valid_start_indices": [],
            }
            for h in range(ix.num_kv_heads):
                lo, hi = int(ix.starts[h, cub[s]]), int(ix.starts[h, cub[s + 1]])
                d["valid_topk_idx_permuted_tile"].append(ix.sel_tokens[h, lo:hi] - cu[s])
                d["valid_lens"].append(lens_all[h])
                d["valid_start_indices"].append(
                    torch.nn.functional.pad(lens_all[h].cumsum(0)[:-1], (1, 0), value=0))
            super().append(d)
        self._built = True

    def __getitem__(self, i):
        self._build()
        return super().__getitem__(i)

    def __len__(self):
        return self.index.batch

    def __iter__(self):
        self._build()
        return super().__iter__()


def _build_kernel_index(topk_idx, cu_seqlens, block_size):
    """Index the kernels run on.  Blocks of 256 keys are handled as pairs of 128-key blocks (the same key set
    for every query); the dicts of `PermuteResults` are still built for the caller's block size."""
    if block_size == 256:
        split = _ops.split_topk_blocks(topk_idx, cu_seqlens, 256, 2)
        return _ops.build_index(split, cu_seqlens, 128), (topk_idx, cu_seqlens, 256)
    return _ops.build_index(topk_idx, cu_seqlens, block_size), None


def _topk_sparse_attention_fwd_opt(
    q: torch.Tensor,  # [total_len, num_q_heads, head_dim]
    k: torch.Tensor,  # [total_len, num_kv_heads, head_dim]
    v: torch.Tensor,  # [total_len, num_kv_heads, head_dim]
    topk_idx: torch.Tensor,  # [num_kv_heads, total_len, topk]
    block_size: int,
    cu_seqlens_q: torch.Tensor,
    cu_seqlens_k: torch.Tensor,
    max_seqlen_q: int,
    max_seqlen_k: int,
    sm_scale: float,
    causal=True,
):
    """(o, lse [Hq, N] fp32 base 2, permute_results); all sequences in one launch set."""
    assert k.dtype == q.dtype and v.dtype == q.dtype
    assert cu_seqlens_q.dtype == torch.int32 and cu_seqlens_k.dtype == torch.int32
    assert block_size in _BLOCK_SIZES
    assert q.shape[1] % k.shape[1] == 0
    assert causal, "selected attention is causal"
    index, ref_args = _build_kernel_index(topk_idx, cu_seqlens_q, block_size)
    o, lse = _ops.selattn_fwd(q, k, v, index, sm_scale)
    return o, lse, PermuteResults(index, ref_args)


def _topk_sparse_attention_bwd_opt(
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
    permute_results,
):
    """(dq, dk, dv); reuses the forward's index when `permute_results` carries it."""
    assert block_size in _BLOCK_SIZES
    index = getattr(permute_results, "index", None)
    if index is None:
        index, _ = _build_kernel_index(topk_idx, cu_seqlens_q, block_size)
    return _ops.selattn_bwd(q, k, v, o, do, lse, index, sm_scale)


class FSATopkSparseAttention(torch.autograd.Function):
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
        o, lse, permute_results = _topk_sparse_attention_fwd_opt(
            q, k, v, topk_idx, block_size, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, sm_scale)
        ctx.save_for_backward(q, k, v, o, lse, cu_seqlens_q, cu_seqlens_k, topk_idx)
        ctx.permute_results = permute_results
        ctx.sm_scale = sm_scale
        ctx.max_seqlen_q = max_seqlen_q
        ctx.max_seqlen_k = max_seqlen_k
        ctx.block_size = block_size
        return o

    @staticmethod
    def backward(ctx, do: torch.Tensor, *args) -> Any:
        q, k, v, o, lse, cu_seqlens_q, cu_seqlens_k, topk_idx = ctx.saved_tensors
        assert ctx.block_size in _BLOCK_SIZES
        dq, dk, dv = _topk_sparse_attention_bwd_opt(
            o, do, lse, q, k, v, topk_idx, ctx.block_size, cu_seqlens_q, cu_seqlens_k,
            ctx.max_seqlen_q, ctx.max_seqlen_k, ctx.sm_scale, ctx.permute_results)
        return dq, dk, dv, None, None, None, None, None, None, None, None


def FSA_topk_sparse_attention(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    topk_idx: torch.Tensor,
    block_size: int,
    cu_seqlens: torch.Tensor,
    softmax_scale: Optional[float] = None,
) -> torch.Tensor:
    """Top-k block sparse attention over packed variable-length sequences.

    Args:
        q: [total_len, num_q_heads, head_dim], bf16 or fp16
        k, v: [total_len, num_kv_heads, head_dim]
        topk_idx: [num_kv_heads, total_len, topk] int32 block ids local to each
            sequence, valid ids first, -1 = padding
        block_size: key/value block size
        cu_seqlens: [batch + 1] int32
        softmax_scale: defaults to 1/sqrt(head_dim)
    Returns:
        attention output [total_len, num_q_heads, head_dim]
    """
    # The kernels derive every per-sequence size on the device, so unlike the
    # reference (:1988) no host synchronisation is needed for max_seqlen.
    return FSATopkSparseAttention.apply(q, k, v, topk_idx, block_size, cu_seqlens, cu_seqlens, None, None,
                                        softmax_scale)
