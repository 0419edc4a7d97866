"""Linear key / value compression under the reference's names (nsa_ref/ops/linear_compress.py:295-502)."""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from fsa_hip import ops as _ops


def compressed_seqlens(cu_seqlens: torch.Tensor, kernel_size: int, kernel_stride: int) -> torch.Tensor:
    """int32 cu_seqlens after compression: floor((len - ks) / stride) + 1, 0 for len < ks."""
    seqlens = cu_seqlens[1:] - cu_seqlens[:-1]
    y = torch.div(seqlens - kernel_size, kernel_stride, rounding_mode="floor") + 1
    y = torch.where(seqlens < kernel_size, torch.zeros_like(y), y)
    out = torch.zeros(cu_seqlens.numel(), dtype=torch.int32, device=cu_seqlens.device)
    out[1:] = torch.cumsum(y, 0)
    return out


class LinearCompress(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, w, pe, cu_seqlens, kernel_size, kernel_stride, y_cu_seqlens, total_y, max_y, max_x):
        assert x.dtype == torch.float16 or x.dtype == torch.bfloat16
        assert x.dtype == w.dtype, f"x dtype: {x.dtype}, w dtype: {w.dtype}"
        assert cu_seqlens.dtype == torch.int32
        total_len, num_heads, head_dim = x.shape
        assert w.shape[0] == num_heads
        assert w.shape[1] == kernel_size * head_dim
        assert w.shape[2] == head_dim
        assert kernel_size % kernel_stride == 0
        assert kernel_size in {16, 32, 64, 128}
        assert head_dim % 8 == 0
        w = w.contiguous()
        pe_c = pe.contiguous() if pe is not None else None
        y = _ops.linear_compress_fwd(x, w, cu_seqlens, y_cu_seqlens, total_y, max_y, kernel_size, kernel_stride, pe_c)
        ctx.save_for_backward(x, w, pe_c if pe_c is not None else x.new_empty(0), cu_seqlens, y_cu_seqlens)
        ctx.has_pe = pe is not None
        ctx.kernel_size, ctx.kernel_stride, ctx.max_x = kernel_size, kernel_stride, max_x
        return y

    @staticmethod
    def backward(ctx, dy):
        x, w, pe, cu_x, cu_y = ctx.saved_tensors
        dx, dw, dpe = _ops.linear_compress_bwd(x, w, dy, cu_x, cu_y, ctx.max_x, ctx.kernel_size, ctx.kernel_stride,
                                               pe if ctx.has_pe else None)
        return dx, dw, dpe, None, None, None, None, None, None, None


def linear_compress(
    x: torch.Tensor,
    w: torch.Tensor,
    cu_seqlens: torch.Tensor,
    kernel_size: int,
    kernel_stride: int,
    pe: Optional[torch.Tensor] = None,
    host_seqlens=None,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Compress keys or values with a strided linear kernel.

    x: [total_len, num_heads, head_dim]; w: [num_heads, kernel_size * head_dim, head_dim];
    pe: optional intra-block positional embedding [num_heads, kernel_size, head_dim] (enters as a bias).
    Returns the compressed states [total_compressed_len, num_heads, head_dim] and their cu_seqlens.
    `host_seqlens` (list of sequence lengths already known on the host) avoids a device read-back."""
    if host_seqlens is None:
        host_seqlens = (cu_seqlens[1:] - cu_seqlens[:-1]).tolist()
    y_lens = [(l - kernel_size) // kernel_stride + 1 if l >= kernel_size else 0 for l in host_seqlens]
    y_cu = compressed_seqlens(cu_seqlens, kernel_size, kernel_stride)
    if pe is not None:
        assert pe.dtype == x.dtype and pe.device == x.device
    y = LinearCompress.apply(x, w, pe, cu_seqlens, kernel_size, kernel_stride, y_cu, sum(y_lens), max(y_lens + [0]),
                             max(host_seqlens + [1]))
    return y, y_cu
