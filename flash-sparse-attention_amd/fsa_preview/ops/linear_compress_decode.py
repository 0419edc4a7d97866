"""Incremental linear compression for decode under the reference's name
(fsa_preview/ops/linear_compress_decode.py:14-76): when the new token completes a compression
window, the compressed token of that window is returned, otherwise None."""
import math

import torch

from fsa_hip import ops as _ops


def _linear_compress_decode(
    new_tokens,  # [1, num_heads, head_dim]
    compress_weight,  # [num_heads, head_dim * kernel_size, head_dim]
    kernel_size,
    kernel_stride,
    intra_block_pe=None,  # [num_heads, kernel_size, head_dim] or None
    prev_total_len=0,
    token_buffer=None,  # most recent tokens before the new one
):
    if token_buffer is None:
        all_tokens = new_tokens
        buffer_start_pos = prev_total_len
    else:
        all_tokens = torch.cat([token_buffer, new_tokens], dim=0)
        buffer_start_pos = prev_total_len - token_buffer.shape[0]
    new_total_len = prev_total_len + 1
    prev_max = math.floor((prev_total_len - kernel_size) / kernel_stride) if prev_total_len >= kernel_size else -1
    new_max = math.floor((new_total_len - kernel_size) / kernel_stride) if new_total_len >= kernel_size else -1
    if new_max <= prev_max:
        return None
    lo = new_max * kernel_stride - buffer_start_pos
    hi = lo + kernel_size
    if lo < 0 or hi > all_tokens.shape[0]:
        return None
    window = all_tokens[lo:hi].contiguous()
    dev = window.device
    cu_x = torch.tensor([0, kernel_size], dtype=torch.int32, device=dev)
    cu_y = torch.tensor([0, 1], dtype=torch.int32, device=dev)
    pe = intra_block_pe.contiguous() if intra_block_pe is not None else None
    # one window: the stride is irrelevant, the window starts at row 0
    return _ops.linear_compress_fwd(window, compress_weight.contiguous(), cu_x, cu_y, 1, 1, kernel_size,
                                    kernel_size, pe)
