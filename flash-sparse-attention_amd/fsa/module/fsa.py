"""`FlashSparseAttention` layer under the reference's name (fsa/module/fsa.py:12-173): same
constructor, parameter names / shapes / initialisation and forward contract.

Branches: compressed attention (+ top-k block selection), selected attention, sliding-window
attention, mixed by a sigmoid gate.  Every attention-side operator runs in the gfx950 library;
the dense projections are torch.nn.Linear (rocBLAS / hipBLASLt), as in the reference."""
from __future__ import annotations

import torch

from fsa.ops import FSA_topk_sparse_attention
from fsa_hip import ops as _ops
from nsa_ref.module.rope import RopeConfig, RotaryEmbedding
from nsa_ref.ops import compressed_attention, linear_compress


class _SlidingWindowAttention(torch.autograd.Function):
    """Causal attention restricted to the last `window` + 1 keys (the reference calls
    flash_attn_varlen_func(causal=True, window_size=(window, -1)), fsa/module/fsa.py:149-159)."""

    @staticmethod
    def forward(ctx, q, k, v, cu_seqlens, max_seqlen, window):
        o, lse = _ops.winattn_fwd(q, k, v, cu_seqlens, max_seqlen, window)
        ctx.save_for_backward(q, k, v, o, lse, cu_seqlens)
        ctx.args = (max_seqlen, window)
        return o

    @staticmethod
    def backward(ctx, do):
        q, k, v, o, lse, cu_seqlens = ctx.saved_tensors
        max_seqlen, window = ctx.args
        dq, dk, dv = _ops.winattn_bwd(q, k, v, o, do, lse, cu_seqlens, max_seqlen, window)
        return dq, dk, dv, None, None, None


class _GateMerge(torch.autograd.Function):
    """Gate-weighted sum of the three branch outputs in one pass (fsa/module/fsa.py:162-167)."""

    @staticmethod
    def forward(ctx, a, b, c, gate):
        ctx.save_for_backward(a, b, c, gate)
        return _ops.gate_merge_fwd(a, b, c, gate)

    @staticmethod
    def backward(ctx, d_out):
        a, b, c, gate = ctx.saved_tensors
        return _ops.gate_merge_bwd(d_out, a, b, c, gate)


class FlashSparseAttention(torch.nn.Module):
    def __init__(
        self,
        hidden_size: int,
        num_q_heads: int,
        num_kv_heads: int,
        head_dim: int,
        kernel_size: int,
        kernel_stride: int,
        block_size: int,
        topk: int,
        init_blocks: int,
        local_blocks: int,
        window_size: int,
        rope_config: RopeConfig,
    ):
        super().__init__()
        self.hidden_size = hidden_size
        self.num_q_heads = num_q_heads
        self.num_kv_heads = num_kv_heads
        self.head_dim = head_dim
        self.kernel_size = kernel_size
        self.kernel_stride = kernel_stride
        self.block_size = block_size
        self.topk = topk
        self.init_blocks = init_blocks
        self.local_blocks = local_blocks
        self.window_size = window_size
        self.rope_config = rope_config

        self.proj_q = torch.nn.Linear(self.hidden_size, self.num_q_heads * self.head_dim, bias=False)
        self.proj_k = torch.nn.Linear(self.hidden_size, self.num_kv_heads * self.head_dim, bias=False)
        self.proj_v = torch.nn.Linear(self.hidden_size, self.num_kv_heads * self.head_dim, bias=False)
        self.proj_o = torch.nn.Linear(self.num_q_heads * self.head_dim, self.hidden_size, bias=False)

        self.compress_key = torch.nn.Parameter(
            torch.zeros(self.num_kv_heads, self.head_dim * self.kernel_size, self.head_dim))
        self.compress_value = torch.nn.Parameter(
            torch.zeros(self.num_kv_heads, self.head_dim * self.kernel_size, self.head_dim))
        self.intra_block_pe = torch.nn.Parameter(torch.zeros(self.num_kv_heads, self.kernel_size, self.head_dim))

        self.gate = torch.nn.Sequential(torch.nn.Linear(self.hidden_size, 3, bias=False), torch.nn.Sigmoid())
        self.rope = RotaryEmbedding(self.rope_config)
        self.init_params()

    def init_params(self):
        for p in self.parameters():
            torch.nn.init.xavier_uniform_(p)

    def forward(
        self,
        x: torch.Tensor,  # [total_len, hidden_size]
        cu_seqlens: torch.Tensor,  # [batch_size + 1]
        return_topk_idx: bool = False,
    ):
        assert x.dtype == torch.bfloat16 or x.dtype == torch.float16
        assert x.shape[-1] == self.hidden_size
        cu_seqlens = cu_seqlens.to(torch.int32)
        # one host read of the sequence lengths serves every size the layer needs
        # (the reference reads back four maxima, fsa/module/fsa.py:121-122,155-156)
        lens = (cu_seqlens[1:] - cu_seqlens[:-1]).tolist()
        max_len = max(lens)
        clens = [(l - self.kernel_size) // self.kernel_stride + 1 if l >= self.kernel_size else 0 for l in lens]

        q = self.proj_q(x).view(-1, self.num_q_heads, self.head_dim)
        k = self.proj_k(x).view(-1, self.num_kv_heads, self.head_dim)
        v = self.proj_v(x).view(-1, self.num_kv_heads, self.head_dim)

        # compressed keys / values are built from the un-rotated k, v
        compressed_k, compressed_cu = linear_compress(k, self.compress_key, cu_seqlens, self.kernel_size,
                                                      self.kernel_stride, self.intra_block_pe, host_seqlens=lens)
        compressed_v, _ = linear_compress(v, self.compress_value, cu_seqlens, self.kernel_size, self.kernel_stride,
                                          None, host_seqlens=lens)

        q = self.rope(q, cu_seqlens)
        compressed_k = self.rope(compressed_k, compressed_cu, start=0, stride=self.kernel_stride)

        compressed_attn_output, topk_idx = compressed_attention(
            q, compressed_k, compressed_v, self.kernel_size, self.kernel_stride, self.block_size, self.topk,
            cu_seqlens, compressed_cu, max_len, max(max(clens), 1), None, self.init_blocks, self.local_blocks,
            parallel_topk_compute=False)

        k = self.rope(k, cu_seqlens)

        # one kernel family serves every GQA group size (the reference switches kernels above 8)
        sparse_attn_output = FSA_topk_sparse_attention(q, k, v, topk_idx, self.block_size, cu_seqlens, None)

        sliding_attn_output = _SlidingWindowAttention.apply(q, k, v, cu_seqlens, max_len, self.window_size)

        gate = self.gate(x)
        attn_output = _GateMerge.apply(compressed_attn_output, sparse_attn_output, sliding_attn_output, gate)
        attn_output = self.proj_o(attn_output.reshape(attn_output.shape[0], -1))
        if return_topk_idx:
            return attn_output, topk_idx
        return attn_output
