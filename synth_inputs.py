"""Synthetic top-k block lists and inputs for benchmarks and tests."""
from __future__ import annotations

import torch


def make_topk_idx(cu_seqlens, num_kv_heads: int, block_size: int, topk: int, seed: int = 0,
                  chunk: int = 8192) -> torch.Tensor:
    """int32 [Hkv, N, T] block lists, one independent draw per kv head.

    For the query at sequence-local position i (own block j = i // B_K): blocks
    {0, j} plus topk-2 distinct blocks drawn uniformly without replacement from
    {1..j-1}; every block 0..j when j + 1 <= topk.  Ascending, -1 padded.
    """
    cu = [int(x) for x in cu_seqlens]
    N = cu[-1]
    gen = torch.Generator().manual_seed(seed)
    out = torch.full((num_kv_heads, N, topk), -1, dtype=torch.int32)
    for s in range(len(cu) - 1):
        s0, s1 = cu[s], cu[s + 1]
        L = s1 - s0
        nblk = (L + block_size - 1) // block_size
        blk = torch.arange(nblk)
        for h in range(num_kv_heads):
            for i0 in range(0, L, chunk):
                i1 = min(L, i0 + chunk)
                j = (torch.arange(i0, i1) // block_size)[:, None]  # [C, 1]
                r = torch.rand(i1 - i0, nblk, generator=gen)
                cand = (blk[None, :] >= 1) & (blk[None, :] < j)
                r = torch.where(cand, r, torch.full_like(r, 2.0))
                r = torch.where(blk[None, :] == 0, torch.full_like(r, -2.0), r)  # block 0 always
                r = torch.where(blk[None, :] == j, torch.full_like(r, -1.0), r)  # own block always
                kk = min(topk, nblk)
                val, idx = torch.topk(r, kk, dim=1, largest=False)
                idx = torch.where(val < 1.5, idx, torch.full_like(idx, nblk + 1))
                idx = idx.sort(dim=1).values
                idx = torch.where(idx > nblk, torch.full_like(idx, -1), idx)
                out[h, s0 + i0 : s0 + i1, :kk] = idx.to(torch.int32)
    return out


def make_qkv(total_len: int, num_q_heads: int, num_kv_heads: int, head_dim: int, dtype, seed: int = 0,
             std: float = 1.0, device="cpu", with_do: bool = True):
    """q, k, v (and dO) ~ N(0, std^2), drawn in fp32 on the CPU from `seed`, then cast."""
    gen = torch.Generator().manual_seed(seed)
    shapes = [(total_len, num_q_heads, head_dim), (total_len, num_kv_heads, head_dim),
              (total_len, num_kv_heads, head_dim)]
    if with_do:
        shapes.append((total_len, num_q_heads, head_dim))
    return tuple((torch.randn(s, generator=gen) * std).to(dtype).to(device) for s in shapes)
