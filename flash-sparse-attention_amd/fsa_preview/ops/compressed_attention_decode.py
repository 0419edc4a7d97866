"""One-step decode of the compressed branch under the reference's name
(fsa_preview/ops/compressed_attention_decode.py:100-207).

The reference handles exactly one request (it asserts a single query row); so does this wrapper,
the batched entry points live in fsa_hip.ops.decode_cmpattn / decode_topk.  `as_written=True`
reproduces the reference's block-score conventions literally (candidate blocks counted from the
compressed length, own block taken as 0, kv head h scored by q-head h); the default scores what
prefill scores for the last token, and ranks the block scores after rounding them to bf16 as the
prefill layer does (scores_to_bf16; the reference's decode ranks fp32 scores, which as_written
keeps).  The returned ids are ordered by descending score."""
import math
import warnings
from typing import Tuple

import torch

from fsa_hip import ops as _ops


def _compressed_attention_decode(
    q: torch.Tensor,  # [1, num_q_heads, head_dim]
    k: torch.Tensor,  # [compressed_len, num_kv_heads, head_dim]
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
    query_start_index: int = 0,
    as_written: bool = False,
    scores_to_bf16: bool = None,
) -> Tuple[torch.Tensor, torch.Tensor]:
    assert q.dtype == torch.bfloat16 or q.dtype == torch.float16
    assert q.dtype == k.dtype and k.dtype == v.dtype
    assert cu_seqlens_q.dtype == torch.int32 and cu_seqlens_k.dtype == torch.int32
    assert q.shape[0] == 1, "one query row per call, as in the reference"
    if sm_scale is None:
        sm_scale = 1 / math.sqrt(q.shape[-1])
    if max_seqlen_k is None:
        max_seqlen_k = k.shape[0]
    dev = q.device
    pos = torch.tensor([query_start_index], dtype=torch.int32, device=dev)
    o, lse, raw = _ops.decode_cmpattn(q, k, v, cu_seqlens_k, pos, kernel_size, kernel_stride, max_seqlen_k, sm_scale,
                                      want_scores=topk > 0, score_head_as_written=as_written)
    if topk <= 0:
        warnings.warn("topk <= 0, returned topk_idx will be None")
        return o, None
    assert topk >= init_blocks + local_blocks
    seqlen = query_start_index + 1
    nblk = math.ceil(max_seqlen_k / block_size) if as_written else math.ceil(seqlen / block_size)
    nblk = max(nblk, 1)
    seqlens = torch.tensor([seqlen], dtype=torch.int32, device=dev)
    idx = _ops.decode_topk(raw, lse, cu_seqlens_k, pos, seqlens, q.shape[1], kernel_size, kernel_stride, block_size,
                           min(topk, nblk), nblk, init_blocks, local_blocks, sm_scale, as_written=as_written,
                           scores_to_bf16=(not as_written) if scores_to_bf16 is None else scores_to_bf16)
    return o, idx  # idx: [num_kv_heads, 1, min(topk, nblk)] int32
