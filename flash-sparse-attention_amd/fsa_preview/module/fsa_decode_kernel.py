"""One decode step of the three attention branches on given q / k / v rows, under the reference's name
(fsa_preview/module/fsa_decode_kernel.py:11-176): same constructor, parameter names and forward arguments.

Steps (one request, one new token, as in the reference): append the new k / v row to the raw cache, extend the
compressed cache when the new token completes a compression window, compressed attention + top-k block selection,
selected attention, sliding-window attention, sigmoid-gated sum.  Every attention runs in the gfx950 decode kernels
behind the C ABI (`fsa_hip.ops.decode_*`); the window branch is the dense decode kernel over the last
window_size + 1 cache rows.

Default semantics are what the prefill layer computes for the same token.  `as_written=True` reproduces the
reference literally where it differs: the compression step is fed the tail of the COMPRESSED cache and its length
(:88-100), block scores use the reference's decode conventions, and the selected branch keeps key 0 only
(fsa_preview/ops/selected_attention_decode.py:29-40 through nsa_ref/ops/topk_sparse_attention.py:116-119,162).
"""
import torch

from fsa_hip import ops as _ops
from fsa_preview.ops import (_compressed_attention_decode, _linear_compress_decode,
                             _topk_sparse_attention_decode)


def decode_step_attention(mod, q, k, v, k_new, v_new, cmp_k, cmp_v, k_rows_for_compress, cu_seqlens_q, cu_seqlens_k,
                          rotate, as_written):
    """Shared by the two decode modules.  q [1, Hq, D]; k, v [L + 1, Hkv, D] raw caches with the new row appended;
    cmp_k, cmp_v compressed caches (un-rotated).  `rotate(x, cu, start, stride)` applies the rotary embedding (identity
    for the kernel-level module).  Returns (compressed, selected, window outputs, new compressed rows or None)."""
    L = k.shape[0] - 1
    dev = q.device
    ks, st = mod.kernel_size, mod.kernel_stride
    if as_written:   # the compressed cache's own tail and length stand in for the raw tokens (:88-112)
        n_buf = min(ks - 1, cmp_k.shape[0])
        buf_k = cmp_k[-n_buf:] if n_buf > 0 else None
        buf_v = cmp_v[-n_buf:] if n_buf > 0 else None
        prev_len = cmp_k.shape[0]
    else:            # the last kernel_size - 1 raw tokens before the new one
        n_buf = min(ks - 1, L)
        buf_k = k_rows_for_compress[L - n_buf:L] if n_buf > 0 else None
        buf_v = v[L - n_buf:L] if n_buf > 0 else None
        prev_len = L
    new_ck = _linear_compress_decode(k_new, mod.compress_key, ks, st, mod.intra_block_pe, prev_len, buf_k)
    new_cv = _linear_compress_decode(v_new, mod.compress_value, ks, st, None, prev_len, buf_v)
    if new_ck is not None:
        compressed_k = torch.cat([cmp_k, new_ck], dim=0)
        compressed_v = torch.cat([cmp_v, new_cv], dim=0)
    else:
        compressed_k, compressed_v = cmp_k, cmp_v
    n_ck = compressed_k.shape[0]
    compressed_cu = torch.tensor([0, n_ck], dtype=torch.int32, device=dev)

    q_r = rotate(q, cu_seqlens_q, 0 if as_written else L, 1)   # the reference rotates the query for position 0
    if n_ck > 0:
        ck_r = rotate(compressed_k, compressed_cu, 0, st)
        cmp_out, topk_idx = _compressed_attention_decode(
            q_r, ck_r, compressed_v, ks, st, mod.block_size, mod.topk, cu_seqlens_q, compressed_cu, 1, n_ck, None,
            mod.init_blocks, mod.local_blocks, query_start_index=L, as_written=as_written)
    else:            # no compressed key yet: the branch contributes nothing; every existing block is selected
        cmp_out = torch.zeros_like(q_r)
        nblk = (L + mod.block_size) // mod.block_size
        ids = torch.arange(min(mod.topk, nblk), dtype=torch.int32, device=dev)
        topk_idx = ids.view(1, 1, -1).expand(mod.num_kv_heads, 1, -1).contiguous()

    k_r = rotate(k, cu_seqlens_k, 0, 1)
    sel_out = _topk_sparse_attention_decode(q_r, k_r, v, topk_idx, mod.block_size, cu_seqlens_q, cu_seqlens_k, 1,
                                            L + 1, None, as_written=as_written)
    # sliding window: the new token attends the last window_size + 1 cache rows, itself included
    # (flash_attn_varlen_func(causal=False, window_size=(w, -1)) with one query row, :153-163)
    w0 = max(0, L - mod.window_size)
    n_win = L + 1 - w0
    cu_w = torch.tensor([0, n_win], dtype=torch.int32, device=dev)
    pos_w = torch.tensor([n_win - 1], dtype=torch.int32, device=dev)
    win_out, _, _ = _ops.decode_cmpattn(q_r, k_r[w0:], v[w0:], cu_w, pos_w, 1, 1, n_win, None, want_scores=False)
    return cmp_out, sel_out, win_out, (new_ck, new_cv)


class FlashSparseAttentionDecodeKernel(torch.nn.Module):
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

        self.compress_key = torch.nn.Parameter(
            torch.zeros(self.num_kv_heads, self.head_dim * self.kernel_size, self.head_dim))
        self.compress_value = torch.nn.Parameter(
            torch.zeros(self.num_kv_heads, self.head_dim * self.kernel_size, self.head_dim))
        self.intra_block_pe = torch.nn.Parameter(torch.zeros(self.num_kv_heads, self.kernel_size, self.head_dim))
        self.gate = torch.nn.Sequential(torch.nn.Linear(self.hidden_size, 3, bias=False), torch.nn.Sigmoid())

    @torch.no_grad()
    def forward(
        self,
        q: torch.Tensor,      # [1, num_q_heads, head_dim]
        k_new: torch.Tensor,  # [1, num_kv_heads, head_dim]
        v_new: torch.Tensor,
        cu_seqlens_q: torch.Tensor,
        cu_seqlens_k: torch.Tensor,  # [2]: the cache with the new token
        k_cache: torch.Tensor = None,
        v_cache: torch.Tensor = None,
        cmp_k_cache: torch.Tensor = None,
        cmp_v_cache: torch.Tensor = None,
        as_written: bool = False,
        return_new_compressed: bool = False,
    ):
        assert q.dtype == torch.bfloat16 or q.dtype == torch.float16
        assert q.shape[0] == 1 and k_new.shape[0] == 1, "one request, one new token per call, as in the reference"
        cu_seqlens_q = cu_seqlens_q.to(torch.int32)
        cu_seqlens_k = cu_seqlens_k.to(torch.int32)
        k = torch.cat([k_cache, k_new], dim=0)
        v = torch.cat([v_cache, v_new], dim=0)
        cmp_out, sel_out, win_out, new_c = decode_step_attention(
            self, q, k, v, k_new, v_new, cmp_k_cache, cmp_v_cache, k, cu_seqlens_q, cu_seqlens_k,
            lambda x, cu, start, stride: x, as_written)
        gate = self.gate(q.reshape(1, -1))
        attn_output = _ops.gate_merge_fwd(cmp_out.reshape(1, -1), sel_out.reshape(1, -1), win_out.reshape(1, -1),
                                          gate.contiguous())
        if return_new_compressed:
            return attn_output, new_c
        return attn_output
