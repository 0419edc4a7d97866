"""Thin Python layer over the C ABI: torch tensors in, raw pointers out.

torch is used for device memory and streams only; every computation happens in
the HIP kernels of libfsa_gfx950.so.
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Optional, Tuple

import torch

from . import _lib

_DTYPE = {torch.bfloat16: 0, torch.float16: 1}


def _ptr(t: Optional[torch.Tensor]):
    return None if t is None else t.data_ptr()


def _stream(device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


def _require_cuda(*tensors):
    for t in tensors:
        if not t.is_cuda:
            raise RuntimeError("fsa_hip: tensors must live on a ROCm device; there is no CPU path")


@dataclass
class SelIndex:
    """Inverted block->query index of one call (all sequences, all kv heads)."""
    cu_seqlens: torch.Tensor   # [B+1] int32
    batch: int
    total_tokens: int
    num_kv_heads: int
    topk: int
    block_size: int
    max_blocks: int            # host upper bound of the number of global blocks
    cu_blocks: torch.Tensor    # [B+1] int32
    counts: torch.Tensor       # [Hkv, max_blocks] int32
    starts: torch.Tensor       # [Hkv, max_blocks+1] int32
    sel_tokens: torch.Tensor   # [Hkv, N*T] int32
    slot_of: torch.Tensor      # [Hkv, N, T] int32


def build_index(topk_idx: torch.Tensor, cu_seqlens: torch.Tensor, block_size: int) -> SelIndex:
    _require_cuda(topk_idx, cu_seqlens)
    assert topk_idx.dtype == torch.int32 and cu_seqlens.dtype == torch.int32
    assert topk_idx.dim() == 3 and topk_idx.stride(2) == 1
    lib = _lib.load()
    hkv, n, t = topk_idx.shape
    batch = cu_seqlens.numel() - 1
    max_blocks = (n + block_size - 1) // block_size + batch
    dev = topk_idx.device
    i32 = dict(dtype=torch.int32, device=dev)
    cu_blocks = torch.empty(batch + 1, **i32)
    counts = torch.empty(hkv, max_blocks, **i32)
    starts = torch.empty(hkv, max_blocks + 1, **i32)
    sel_tokens = torch.empty(hkv, n * t, **i32)
    slot_of = torch.empty(hkv, n, t, **i32)
    ws_bytes = lib.fsa_index_workspace_bytes(n, t, hkv, max_blocks)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    rc = lib.fsa_build_index(_ptr(topk_idx), topk_idx.stride(0), topk_idx.stride(1), _ptr(cu_seqlens),
                             batch, n, hkv, t, block_size, max_blocks, _ptr(cu_blocks), _ptr(counts),
                             _ptr(starts), _ptr(sel_tokens), _ptr(slot_of), _ptr(ws), ws_bytes,
                             _stream(dev))
    _lib.check(rc, "fsa_build_index")
    return SelIndex(cu_seqlens, batch, n, hkv, t, block_size, max_blocks, cu_blocks, counts, starts,
                    sel_tokens, slot_of)


def _check_qkv(q, k, v):
    _require_cuda(q, k, v)
    assert q.dtype in _DTYPE, "q must be bf16 or fp16"
    assert q.dtype == k.dtype == v.dtype
    assert q.dim() == 3 and k.dim() == 3 and v.dim() == 3
    assert q.stride(2) == 1 and k.stride(2) == 1 and v.stride(2) == 1
    assert q.shape[1] % k.shape[1] == 0
    assert k.shape == v.shape and q.shape[0] == k.shape[0] and q.shape[2] == k.shape[2]


def selattn_fwd(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, index: SelIndex,
                softmax_scale: Optional[float] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """Selected attention forward: returns (o [N,Hq,D], lse [Hq,N] fp32 base 2)."""
    _check_qkv(q, k, v)
    lib = _lib.load()
    n, hq, d = q.shape
    hkv = k.shape[1]
    assert hkv == index.num_kv_heads and n == index.total_tokens
    if softmax_scale is None:
        softmax_scale = 1.0 / math.sqrt(d)
    dev = q.device
    o = torch.empty((n, hq, d), dtype=q.dtype, device=dev)
    lse = torch.empty((hq, n), dtype=torch.float32, device=dev)
    ws_bytes = lib.fsa_selattn_fwd_workspace_bytes(n, hq, hkv, d, index.topk, index.max_blocks)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    rc = lib.fsa_selattn_fwd(
        _ptr(q), _ptr(k), _ptr(v), _DTYPE[q.dtype],
        q.stride(0), q.stride(1), k.stride(0), k.stride(1), v.stride(0), v.stride(1),
        _ptr(index.cu_seqlens), index.batch, n, hq, hkv, d, index.topk, index.block_size,
        index.max_blocks, float(softmax_scale),
        _ptr(index.cu_blocks), _ptr(index.counts), _ptr(index.starts), _ptr(index.sel_tokens),
        _ptr(index.slot_of),
        _ptr(o), o.stride(0), o.stride(1), _ptr(lse), _ptr(ws), ws_bytes, _stream(dev))
    _lib.check(rc, "fsa_selattn_fwd")
    return o, lse


def selattn_bwd(q, k, v, o, do, lse, index: SelIndex, softmax_scale: Optional[float] = None):
    """Selected attention backward: returns (dq, dk, dv) in the input dtype."""
    _check_qkv(q, k, v)
    _require_cuda(o, do, lse)
    assert o.dtype == q.dtype and do.dtype == q.dtype and lse.dtype == torch.float32
    assert o.shape == q.shape and do.shape == q.shape
    lib = _lib.load()
    n, hq, d = q.shape
    hkv = k.shape[1]
    if softmax_scale is None:
        softmax_scale = 1.0 / math.sqrt(d)
    if do.stride(2) != 1:
        do = do.contiguous()
    if o.stride(2) != 1:
        o = o.contiguous()
    lse = lse.contiguous()
    dev = q.device
    dq = torch.empty((n, hq, d), dtype=q.dtype, device=dev)
    dk = torch.empty((n, hkv, d), dtype=q.dtype, device=dev)
    dv = torch.empty((n, hkv, d), dtype=q.dtype, device=dev)
    ws_bytes = lib.fsa_selattn_bwd_workspace_bytes(n, hq, hkv, d, index.topk, index.block_size,
                                                   index.max_blocks)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    rc = lib.fsa_selattn_bwd(
        _ptr(q), _ptr(k), _ptr(v), _ptr(o), _ptr(do), _ptr(lse), _DTYPE[q.dtype],
        q.stride(0), q.stride(1), k.stride(0), k.stride(1), v.stride(0), v.stride(1),
        o.stride(0), o.stride(1), do.stride(0), do.stride(1),
        _ptr(index.cu_seqlens), index.batch, n, hq, hkv, d, index.topk, index.block_size,
        index.max_blocks, float(softmax_scale),
        _ptr(index.cu_blocks), _ptr(index.counts), _ptr(index.starts), _ptr(index.sel_tokens),
        _ptr(index.slot_of),
        _ptr(dq), _ptr(dk), _ptr(dv), _ptr(ws), ws_bytes, _stream(dev))
    _lib.check(rc, "fsa_selattn_bwd")
    return dq, dk, dv
