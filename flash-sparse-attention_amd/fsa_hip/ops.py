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


# Head dims the kernels are built for.  Any other head_dim <= 256 (the reference accepts every head_dim <= 256,
# README.md:63, by padding tiles to the next power of two inside its kernels) runs on the next built size with
# zero-padded rows: q.k and P.V are unchanged by zero columns, the softmax scale is taken from the true head_dim,
# and the padded columns of the outputs and gradients are cut off again.
_NATIVE_D = (64, 128, 256)


def _native_dim(d: int, native=_NATIVE_D) -> int:
    for nd in native:
        if d <= nd:
            return nd
    raise ValueError(f"head_dim {d} is not supported (at most {native[-1]})")


def _resize_d(t: torch.Tensor, d_to: int) -> torch.Tensor:
    """[..., H, d] -> contiguous [..., H, d_to]: the leading columns copied, the rest zero (fsa_pad_head_dim)."""
    d = t.shape[-1]
    rows = t.reshape(-1, t.shape[-2], d) if t.dim() != 3 else t
    if (t.numel() == 0 or t.dtype not in _DTYPE or not t.is_cuda or rows.stride(2) != 1 or d % 4 or d_to % 4
            or rows.stride(0) % 4 or rows.stride(1) % 4 or t.data_ptr() % 8):
        # what the C helper does not take (empty tensors, fp32 gradients of parameters, odd head dims): torch copies
        return (torch.nn.functional.pad(t, (0, d_to - d)) if d_to > d else t[..., :d_to]).contiguous()
    out = torch.empty((*t.shape[:-1], d_to), dtype=t.dtype, device=t.device)
    o3 = out.view(-1, t.shape[-2], d_to)
    rc = _lib.load().fsa_pad_head_dim(_ptr(rows), rows.stride(0), rows.stride(1), d, _ptr(o3), o3.stride(0),
                                      o3.stride(1), d_to, rows.shape[0], rows.shape[1], _stream(t.device))
    _lib.check(rc, "fsa_pad_head_dim")
    return out


def _pad_d(t: Optional[torch.Tensor], d_to: int):
    if t is None or t.shape[-1] == d_to:
        return t
    return _resize_d(t, d_to)


def _cut_d(t: torch.Tensor, d: int):
    return _resize_d(t, d) if t.shape[-1] != d else t


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


def split_topk_blocks(topk_idx: torch.Tensor, cu_seqlens: torch.Tensor, block_size: int, factor: int) -> torch.Tensor:
    """topk_idx over blocks of `block_size` keys -> [Hkv, N, T*factor] over blocks of block_size // factor keys
    (sub-blocks that start after the query become -1); the selected key set of every query is unchanged."""
    _require_cuda(topk_idx, cu_seqlens)
    assert topk_idx.dtype == torch.int32 and cu_seqlens.dtype == torch.int32
    assert topk_idx.dim() == 3 and topk_idx.stride(2) == 1
    lib = _lib.load()
    hkv, n, t = topk_idx.shape
    out = torch.empty((hkv, n, t * factor), dtype=torch.int32, device=topk_idx.device)
    rc = lib.fsa_split_topk_blocks(_ptr(topk_idx), topk_idx.stride(0), topk_idx.stride(1), _ptr(cu_seqlens),
                                   cu_seqlens.numel() - 1, n, hkv, t, block_size, factor, _ptr(out),
                                   _stream(topk_idx.device))
    _lib.check(rc, "fsa_split_topk_blocks")
    return out


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
    dn = _native_dim(d)
    if dn != d:
        o, lse = selattn_fwd(_pad_d(q, dn), _pad_d(k, dn), _pad_d(v, dn), index, softmax_scale)
        return _cut_d(o, d), lse
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
    dn = _native_dim(d)
    if dn != d:
        g = selattn_bwd(_pad_d(q, dn), _pad_d(k, dn), _pad_d(v, dn), _pad_d(o, dn), _pad_d(do, dn), lse, index,
                        softmax_scale)
        return tuple(_cut_d(t, d) for t in g)
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


def _check_cmp(q, ck, cv, cu_q, cu_k):
    _require_cuda(q, ck, cv, cu_q, cu_k)
    assert q.dtype in _DTYPE and q.dtype == ck.dtype == cv.dtype
    assert cu_q.dtype == torch.int32 and cu_k.dtype == torch.int32
    assert q.stride(2) == 1 and ck.stride(2) == 1 and cv.stride(2) == 1
    assert ck.shape == cv.shape and q.shape[1] % ck.shape[1] == 0 and q.shape[2] == ck.shape[2]


def cmpattn_fwd(q, ck, cv, kernel_size, kernel_stride, cu_q, cu_k, max_seqlen_q, softmax_scale=None):
    """Compressed attention forward: (o [N,Hq,D], lse [Hq,N] fp32 base 2)."""
    _check_cmp(q, ck, cv, cu_q, cu_k)
    lib = _lib.load()
    n, hq, d = q.shape
    hkv = ck.shape[1]
    if softmax_scale is None:
        softmax_scale = 1.0 / math.sqrt(d)
    dn = _native_dim(d)
    if dn != d:
        o, lse = cmpattn_fwd(_pad_d(q, dn), _pad_d(ck, dn), _pad_d(cv, dn), kernel_size, kernel_stride, cu_q, cu_k,
                             max_seqlen_q, softmax_scale)
        return _cut_d(o, d), lse
    o = torch.empty_like(q)
    lse = torch.empty((hq, n), dtype=torch.float32, device=q.device)
    if ck.shape[0] == 0:
        return o.zero_(), lse.fill_(float("-inf"))
    rc = lib.fsa_cmpattn_fwd(_ptr(q), _ptr(ck), _ptr(cv), _DTYPE[q.dtype], q.stride(0), q.stride(1),
                             ck.stride(0), ck.stride(1), cv.stride(0), cv.stride(1), _ptr(cu_q), _ptr(cu_k),
                             cu_q.numel() - 1, n, int(max_seqlen_q), hq, hkv, d, kernel_size, kernel_stride,
                             float(softmax_scale), _ptr(o), o.stride(0), o.stride(1), _ptr(lse),
                             _stream(q.device))
    _lib.check(rc, "fsa_cmpattn_fwd")
    return o, lse


def cmpattn_bwd(q, ck, cv, o, do, lse, kernel_size, kernel_stride, cu_q, cu_k, max_seqlen_q,
                softmax_scale=None):
    """Compressed attention backward: (dq, dck, dcv)."""
    _check_cmp(q, ck, cv, cu_q, cu_k)
    lib = _lib.load()
    n, hq, d = q.shape
    nk, hkv, _ = ck.shape
    if softmax_scale is None:
        softmax_scale = 1.0 / math.sqrt(d)
    dn = _native_dim(d)
    if dn != d:
        g = cmpattn_bwd(_pad_d(q, dn), _pad_d(ck, dn), _pad_d(cv, dn), _pad_d(o, dn), _pad_d(do, dn), lse, kernel_size,
                        kernel_stride, cu_q, cu_k, max_seqlen_q, softmax_scale)
        return tuple(_cut_d(t, d) for t in g)
    if do.stride(2) != 1:
        do = do.contiguous()
    dq = torch.empty((n, hq, d), dtype=q.dtype, device=q.device)
    dck = torch.empty((nk, hkv, d), dtype=q.dtype, device=q.device)
    dcv = torch.empty((nk, hkv, d), dtype=q.dtype, device=q.device)
    if nk == 0:
        return dq.zero_(), dck, dcv
    batch = cu_q.numel() - 1
    ws_bytes = lib.fsa_cmpattn_bwd_workspace_bytes(n, nk, int(max_seqlen_q), batch, hq, hkv, d)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=q.device)
    rc = lib.fsa_cmpattn_bwd(_ptr(q), _ptr(ck), _ptr(cv), _ptr(o), _ptr(do), _ptr(lse), _DTYPE[q.dtype],
                             q.stride(0), q.stride(1), ck.stride(0), ck.stride(1), cv.stride(0), cv.stride(1),
                             o.stride(0), o.stride(1), do.stride(0), do.stride(1), _ptr(cu_q), _ptr(cu_k),
                             batch, n, nk, int(max_seqlen_q), hq, hkv, d, kernel_size, kernel_stride,
                             float(softmax_scale), _ptr(dq), _ptr(dck), _ptr(dcv), _ptr(ws), ws_bytes,
                             _stream(q.device))
    _lib.check(rc, "fsa_cmpattn_bwd")
    return dq, dck, dcv


def cmp_topk(q, ck, lse, kernel_size, kernel_stride, block_size, topk, cu_q, cu_k, max_seqlen_q,
             max_seqlen_k, init_blocks=1, local_blocks=2, softmax_scale=None, scores_to_bf16=True,
             return_block_score=False, score_head_as_written=False):
    """Top-k block ids [Hkv, N, min(topk, nblk)] int32 from the compressed-attention probabilities of the first
    q head of every group (score_head_as_written: of q head kh for kv head kh, the literal behaviour of the
    reference's parallel path, nsa_ref/ops/compressed_attention.py:870, 898, 906)."""
    _require_cuda(q, ck, lse, cu_q, cu_k)
    lib = _lib.load()
    n, hq, d = q.shape
    hkv = ck.shape[1]
    if softmax_scale is None:
        softmax_scale = 1.0 / math.sqrt(d)
    dn = _native_dim(d)
    if dn != d:
        return cmp_topk(_pad_d(q, dn), _pad_d(ck, dn), lse, kernel_size, kernel_stride, block_size, topk, cu_q, cu_k,
                        max_seqlen_q, max_seqlen_k, init_blocks, local_blocks, softmax_scale, scores_to_bf16,
                        return_block_score, score_head_as_written)
    nblk = (int(max_seqlen_q) + block_size - 1) // block_size
    t_out = min(topk, nblk)
    dev = q.device
    if ck.shape[0] == 0:   # no compressed key in the whole batch: the lengths in cu_k are zero, this row is never read
        ck = torch.zeros((1, hkv, d), dtype=q.dtype, device=dev)
    idx = torch.empty((hkv, n, t_out), dtype=torch.int32, device=dev)
    bscore = torch.empty((hkv, n, nblk), dtype=torch.float32, device=dev) if return_block_score else None
    score_cols = max(1, int(max_seqlen_k))
    if kernel_size == 2 * kernel_stride and block_size == 4 * kernel_stride:
        score_cols = score_cols // 4 + 1  # block scores instead of per-key probabilities
    ws_bytes = lib.fsa_cmp_topk_workspace_bytes(n, hkv, score_cols)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    lse = lse.contiguous()
    rc = lib.fsa_cmp_topk(_ptr(q), _ptr(ck), _ptr(lse), _DTYPE[q.dtype], q.stride(0), q.stride(1),
                          ck.stride(0), ck.stride(1), _ptr(cu_q), _ptr(cu_k), cu_q.numel() - 1, n,
                          int(max_seqlen_q), max(1, int(max_seqlen_k)), hq, hkv, d, kernel_size, kernel_stride,
                          block_size, topk, init_blocks, local_blocks, 1 if scores_to_bf16 else 0,
                          1 if score_head_as_written else 0,
                          float(softmax_scale), _ptr(idx), _ptr(bscore), _ptr(ws), ws_bytes, _stream(dev))
    _lib.check(rc, "fsa_cmp_topk")
    return (idx, bscore) if return_block_score else idx


def decode_cmpattn(q, ck, cv, cu_ck, pos, kernel_size, kernel_stride, max_ck, softmax_scale=None,
                   want_scores=True, score_head_as_written=False):
    """Decode-step compressed attention for a batch of requests.

    q [B,Hq,D]; ck/cv [total_ck,Hkv,D] with cu_ck [B+1]; pos [B] int32 query positions;
    max_ck: host upper bound of the longest compressed cache.
    Returns (o [B,Hq,D], lse [Hq,B], raw_score [Hkv,B,ld] or None)."""
    _require_cuda(q, ck, cv, cu_ck, pos)
    assert q.dtype in _DTYPE and q.dtype == ck.dtype == cv.dtype
    assert q.dim() == 3 and q.stride(2) == 1 and ck.stride(2) == 1 and cv.stride(2) == 1
    lib = _lib.load()
    b, hq, d = q.shape
    hkv = ck.shape[1]
    if softmax_scale is None:
        softmax_scale = 1.0 / math.sqrt(d)
    dn = _native_dim(d)
    if dn != d:
        o, lse, raw = decode_cmpattn(_pad_d(q, dn), _pad_d(ck, dn), _pad_d(cv, dn), cu_ck, pos, kernel_size,
                                     kernel_stride, max_ck, softmax_scale, want_scores, score_head_as_written)
        return _cut_d(o, d), lse, raw
    dev = q.device
    o = torch.empty((b, hq, d), dtype=q.dtype, device=dev)
    lse = torch.empty((hq, b), dtype=torch.float32, device=dev)
    ld = (max(int(max_ck), 1) + 3) // 4 * 4
    raw = torch.empty((hkv, b, ld), dtype=torch.float32, device=dev) if want_scores else None
    max_keys = max(int(max_ck), 0)
    ws_bytes = max(256, lib.fsa_decode_workspace_bytes(b, hq, hkv, d, max_keys))
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    rc = lib.fsa_decode_cmpattn(_ptr(q), _ptr(ck), _ptr(cv), _DTYPE[q.dtype], q.stride(0), q.stride(1),
                                ck.stride(0), ck.stride(1), cv.stride(0), cv.stride(1), _ptr(cu_ck), _ptr(pos),
                                b, hq, hkv, d, kernel_size, kernel_stride, float(softmax_scale),
                                1 if score_head_as_written else 0, max_keys, _ptr(o), _ptr(lse), _ptr(raw), ld,
                                _ptr(ws), ws_bytes, _stream(dev))
    _lib.check(rc, "fsa_decode_cmpattn")
    return o, lse, raw


def decode_topk(raw_score, lse, cu_ck, pos, seqlens, num_q_heads, kernel_size, kernel_stride, block_size,
                topk, max_blocks, init_blocks=1, local_blocks=2, softmax_scale=1.0, as_written=False,
                return_block_score=False, scores_to_bf16=False):
    """Top-k block ids [Hkv,B,topk] int32 (descending score) for the decode step; scores_to_bf16 ranks the block
    scores after rounding them to bf16 (what the prefill selection of the layer does)."""
    _require_cuda(raw_score, lse, cu_ck, pos, seqlens)
    lib = _lib.load()
    hkv, b, ld = raw_score.shape
    dev = raw_score.device
    idx = torch.empty((hkv, b, topk), dtype=torch.int32, device=dev)
    bscore = torch.empty((hkv, b, max_blocks), dtype=torch.float32, device=dev) if return_block_score else None
    rc = lib.fsa_decode_topk(_ptr(raw_score), ld, _ptr(lse), _ptr(cu_ck), _ptr(pos), _ptr(seqlens), b,
                             num_q_heads, hkv, kernel_size, kernel_stride, block_size, topk, init_blocks,
                             local_blocks, 1 if as_written else 0, 1 if scores_to_bf16 else 0,
                             float(softmax_scale), int(max_blocks),
                             _ptr(idx), _ptr(bscore), _stream(dev))
    _lib.check(rc, "fsa_decode_topk")
    return (idx, bscore) if return_block_score else idx


def decode_selattn(q, k_cache, v_cache, cu_k, topk_idx, block_size, softmax_scale=None, seqlens=None):
    """Decode-step selected attention: (o [B,Hq,D], lse [Hq,B]).  `seqlens` (optional, int32 [B] on the device):
    valid rows of each request's slot [cu_k[b], cu_k[b+1]) of the caches; default: the whole slot."""
    _require_cuda(q, k_cache, v_cache, cu_k, topk_idx)
    assert seqlens is None or (seqlens.is_cuda and seqlens.dtype == torch.int32 and seqlens.numel() == q.shape[0])
    assert q.dtype in _DTYPE and q.dtype == k_cache.dtype == v_cache.dtype
    assert topk_idx.dtype == torch.int32 and topk_idx.is_contiguous()
    assert q.stride(2) == 1 and k_cache.stride(2) == 1 and v_cache.stride(2) == 1
    lib = _lib.load()
    b, hq, d = q.shape
    hkv = k_cache.shape[1]
    assert topk_idx.shape[0] == hkv and topk_idx.shape[1] == b
    if softmax_scale is None:
        softmax_scale = 1.0 / math.sqrt(d)
    dn = _native_dim(d)
    if dn != d:
        o, lse = decode_selattn(_pad_d(q, dn), _pad_d(k_cache, dn), _pad_d(v_cache, dn), cu_k, topk_idx, block_size,
                                softmax_scale, seqlens)
        return _cut_d(o, d), lse
    dev = q.device
    o = torch.empty((b, hq, d), dtype=q.dtype, device=dev)
    lse = torch.empty((hq, b), dtype=torch.float32, device=dev)
    topk = topk_idx.shape[2]
    ws_bytes = max(256, lib.fsa_decode_workspace_bytes(b, hq, hkv, d, topk * ((block_size + 31) // 32) * 32))
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    rc = lib.fsa_decode_selattn(_ptr(q), _ptr(k_cache), _ptr(v_cache), _DTYPE[q.dtype], q.stride(0), q.stride(1),
                                k_cache.stride(0), k_cache.stride(1), v_cache.stride(0), v_cache.stride(1),
                                _ptr(cu_k), _ptr(seqlens), _ptr(topk_idx), b, hq, hkv, d, topk_idx.shape[2], block_size,
                                float(softmax_scale), _ptr(o), _ptr(lse), _ptr(ws), ws_bytes, _stream(dev))
    _lib.check(rc, "fsa_decode_selattn")
    return o, lse


def decode_selattn_static(q, k_cache, v_cache, cu_k, topk_idx, block_size, o, lse, softmax_scale=None, seqlens=None):
    """Decode-step selected attention into caller-provided `o` [B,Hq,D] and `lse` [Hq,B], with the partial results
    in the library's built-in scratch buffer: the call allocates nothing (C entry point fsa_decode_selattn_static).
    Raises if the sizes exceed the buffer."""
    _require_cuda(q, k_cache, v_cache, cu_k, topk_idx, o, lse)
    assert q.dtype in _DTYPE and q.dtype == k_cache.dtype == v_cache.dtype == o.dtype
    assert topk_idx.dtype == torch.int32 and topk_idx.is_contiguous()
    assert q.stride(2) == 1 and k_cache.stride(2) == 1 and v_cache.stride(2) == 1
    assert o.is_contiguous() and lse.is_contiguous() and lse.dtype == torch.float32
    lib = _lib.load()
    b, hq, d = q.shape
    hkv = k_cache.shape[1]
    assert topk_idx.shape[0] == hkv and topk_idx.shape[1] == b
    assert o.shape == (b, hq, d) and lse.shape == (hq, b)
    if softmax_scale is None:
        softmax_scale = 1.0 / math.sqrt(d)
    rc = lib.fsa_decode_selattn_static(_ptr(q), _ptr(k_cache), _ptr(v_cache), _DTYPE[q.dtype], q.stride(0),
                                       q.stride(1), k_cache.stride(0), k_cache.stride(1), v_cache.stride(0),
                                       v_cache.stride(1), _ptr(cu_k), _ptr(seqlens), _ptr(topk_idx), b, hq, hkv, d,
                                       topk_idx.shape[2], block_size, float(softmax_scale), _ptr(o), _ptr(lse),
                                       _stream(q.device))
    _lib.check(rc, "fsa_decode_selattn_static")
    return o, lse


def winattn_fwd(q, k, v, cu_seqlens, max_seqlen, window, softmax_scale=None):
    """Causal sliding-window attention (keys i-window..i): (o, lse [Hq,N] fp32 base 2)."""
    _check_qkv(q, k, v)
    lib = _lib.load()
    n, hq, d = q.shape
    hkv = k.shape[1]
    if softmax_scale is None:
        softmax_scale = 1.0 / math.sqrt(d)
    dn = _native_dim(d)
    if dn != d:
        o, lse = winattn_fwd(_pad_d(q, dn), _pad_d(k, dn), _pad_d(v, dn), cu_seqlens, max_seqlen, window, softmax_scale)
        return _cut_d(o, d), lse
    o = torch.empty((n, hq, d), dtype=q.dtype, device=q.device)
    lse = torch.empty((hq, n), dtype=torch.float32, device=q.device)
    rc = lib.fsa_winattn_fwd(_ptr(q), _ptr(k), _ptr(v), _DTYPE[q.dtype], q.stride(0), q.stride(1), k.stride(0),
                             k.stride(1), v.stride(0), v.stride(1), _ptr(cu_seqlens), cu_seqlens.numel() - 1, n,
                             int(max_seqlen), hq, hkv, d, int(window), float(softmax_scale), _ptr(o), o.stride(0),
                             o.stride(1), _ptr(lse), _stream(q.device))
    _lib.check(rc, "fsa_winattn_fwd")
    return o, lse


def winattn_bwd(q, k, v, o, do, lse, cu_seqlens, max_seqlen, window, softmax_scale=None):
    """Backward of winattn_fwd: (dq, dk, dv)."""
    _check_qkv(q, k, v)
    lib = _lib.load()
    n, hq, d = q.shape
    hkv = k.shape[1]
    if softmax_scale is None:
        softmax_scale = 1.0 / math.sqrt(d)
    dn = _native_dim(d)
    if dn != d:
        g = winattn_bwd(_pad_d(q, dn), _pad_d(k, dn), _pad_d(v, dn), _pad_d(o, dn), _pad_d(do, dn), lse, cu_seqlens,
                        max_seqlen, window, softmax_scale)
        return tuple(_cut_d(t, d) for t in g)
    if do.stride(2) != 1:
        do = do.contiguous()
    dev = q.device
    dq = torch.empty((n, hq, d), dtype=q.dtype, device=dev)
    dk = torch.empty((n, hkv, d), dtype=q.dtype, device=dev)
    dv = torch.empty((n, hkv, d), dtype=q.dtype, device=dev)
    batch = cu_seqlens.numel() - 1
    ws_bytes = lib.fsa_winattn_bwd_workspace_bytes(n, int(max_seqlen), int(window), batch, hq, hkv, d)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    rc = lib.fsa_winattn_bwd(_ptr(q), _ptr(k), _ptr(v), _ptr(o), _ptr(do), _ptr(lse), _DTYPE[q.dtype],
                             q.stride(0), q.stride(1), k.stride(0), k.stride(1), v.stride(0), v.stride(1),
                             o.stride(0), o.stride(1), do.stride(0), do.stride(1), _ptr(cu_seqlens), batch, n,
                             int(max_seqlen), hq, hkv, d, int(window), float(softmax_scale), _ptr(dq), _ptr(dk),
                             _ptr(dv), _ptr(ws), ws_bytes, _stream(dev))
    _lib.check(rc, "fsa_winattn_bwd")
    return dq, dk, dv


def rope(x, cu_seqlens, inv_freq, attention_scaling=1.0, start=0, stride=1, inverse=False):
    """Rotary embedding on packed sequences; inverse=True is the backward rotation."""
    _require_cuda(x, cu_seqlens, inv_freq)
    assert x.dtype in _DTYPE and x.dim() == 3 and x.stride(2) == 1
    assert inv_freq.dtype == torch.float32 and inv_freq.numel() == x.shape[2] // 2
    lib = _lib.load()
    n, h, d = x.shape
    out = torch.empty((n, h, d), dtype=x.dtype, device=x.device)
    rc = lib.fsa_rope(_ptr(x), _ptr(out), _DTYPE[x.dtype], x.stride(0), x.stride(1), out.stride(0), out.stride(1),
                      _ptr(cu_seqlens), cu_seqlens.numel() - 1, n, h, d, _ptr(inv_freq.contiguous()),
                      float(attention_scaling), int(start), int(stride), 1 if inverse else 0, _stream(x.device))
    _lib.check(rc, "fsa_rope")
    return out


def _pad_compress_weight(w, kernel_size: int, d: int, dn: int):
    """w [H, ks*d, d] as [H, ks*dn, dn] with zero rows / columns for the padded dims."""
    h = w.shape[0]
    w4 = torch.nn.functional.pad(w.view(h, kernel_size, d, d), (0, dn - d, 0, dn - d))
    return w4.reshape(h, kernel_size * dn, dn).contiguous()


def linear_compress_fwd(x, w, cu_x, cu_y, total_y, max_y, kernel_size, kernel_stride, pe=None):
    """y [total_y, H, D] = strided-window projection of x [N, H, D] with w [H, ks*D, D] (+ pe bias)."""
    _require_cuda(x, w, cu_x, cu_y)
    assert x.dtype in _DTYPE and x.dtype == w.dtype and x.stride(2) == 1 and w.is_contiguous()
    lib = _lib.load()
    n, h, d = x.shape
    dn = _native_dim(d)
    if dn != d:
        y = linear_compress_fwd(_pad_d(x, dn), _pad_compress_weight(w, kernel_size, d, dn), cu_x, cu_y, total_y, max_y,
                                kernel_size, kernel_stride, None if pe is None else _pad_d(pe, dn).contiguous())
        return _cut_d(y, d)
    y = torch.empty((int(total_y), h, d), dtype=x.dtype, device=x.device)
    bias = torch.empty((h, d), dtype=x.dtype, device=x.device) if pe is not None else None
    if pe is not None:
        assert pe.dtype == x.dtype and pe.is_contiguous()
    if total_y > 0:
        rc = lib.fsa_linear_compress_fwd(_ptr(x), _ptr(w), _ptr(pe), _DTYPE[x.dtype], x.stride(0), x.stride(1),
                                         _ptr(cu_x), _ptr(cu_y), cu_x.numel() - 1, int(max_y), h, d, kernel_size,
                                         kernel_stride, _ptr(y), _ptr(bias), _stream(x.device))
        _lib.check(rc, "fsa_linear_compress_fwd")
    return y


def linear_compress_bwd(x, w, dy, cu_x, cu_y, max_x, kernel_size, kernel_stride, pe=None):
    """(dx, dw, dpe or None) of linear_compress_fwd."""
    _require_cuda(x, w, dy, cu_x, cu_y)
    lib = _lib.load()
    n, h, d = x.shape
    dn = _native_dim(d, (128, 256))   # the weight-gradient kernel works on 128 input dims per work-group
    if dn != d:
        dx, dw, dpe = linear_compress_bwd(_pad_d(x, dn), _pad_compress_weight(w, kernel_size, d, dn), _pad_d(dy, dn),
                                          cu_x, cu_y, max_x, kernel_size, kernel_stride,
                                          None if pe is None else _pad_d(pe, dn).contiguous())
        dw = dw.view(h, kernel_size, dn, dn)[:, :, :d, :d].reshape(h, kernel_size * d, d).contiguous()
        return _cut_d(dx, d), dw, (None if dpe is None else _cut_d(dpe, d))
    dev = x.device
    dy = dy.contiguous()
    dx = torch.empty((n, h, d), dtype=x.dtype, device=dev)
    dw = torch.empty_like(w)
    dpe = torch.empty_like(pe) if pe is not None else None
    dbias = torch.empty((h, d), dtype=torch.float32, device=dev) if pe is not None else None
    if dy.shape[0] == 0:
        return dx.zero_(), dw.zero_(), (dpe.zero_() if dpe is not None else None)
    rc = lib.fsa_linear_compress_bwd(_ptr(x), _ptr(w), _ptr(pe), _ptr(dy), _DTYPE[x.dtype], x.stride(0),
                                     x.stride(1), _ptr(cu_x), _ptr(cu_y), cu_x.numel() - 1, int(max_x),
                                     dy.shape[0], h, d, kernel_size, kernel_stride, _ptr(dx), _ptr(dw), _ptr(dpe),
                                     _ptr(dbias), _stream(dev))
    _lib.check(rc, "fsa_linear_compress_bwd")
    return dx, dw, dpe


def gate_merge_fwd(a, b, c, gate):
    """out = gate[:,0] a + gate[:,1] b + gate[:,2] c for a, b, c [N, H, D] and gate [N, 3], one pass."""
    _require_cuda(a, b, c, gate)
    assert a.dtype in _DTYPE and a.dtype == b.dtype == c.dtype == gate.dtype
    assert a.shape == b.shape == c.shape and gate.shape == (a.shape[0], 3)
    a, b, c, gate = (t.contiguous() for t in (a, b, c, gate))
    n = a.shape[0]
    row = a.numel() // max(n, 1)
    out = torch.empty_like(a)
    rc = _lib.load().fsa_gate_merge_fwd(_ptr(a), _ptr(b), _ptr(c), _ptr(gate), _DTYPE[a.dtype], n, row, _ptr(out),
                                        _stream(a.device))
    _lib.check(rc, "fsa_gate_merge_fwd")
    return out


def gate_merge_bwd(d_out, a, b, c, gate):
    """(d_a, d_b, d_c, d_gate) of gate_merge_fwd."""
    _require_cuda(d_out, a, b, c, gate)
    d_out, a, b, c, gate = (t.contiguous() for t in (d_out, a, b, c, gate))
    n = a.shape[0]
    row = a.numel() // max(n, 1)
    d_a, d_b, d_c, d_gate = torch.empty_like(a), torch.empty_like(b), torch.empty_like(c), torch.empty_like(gate)
    rc = _lib.load().fsa_gate_merge_bwd(_ptr(d_out), _ptr(a), _ptr(b), _ptr(c), _ptr(gate), _DTYPE[a.dtype], n, row,
                                        _ptr(d_a), _ptr(d_b), _ptr(d_c), _ptr(d_gate), _stream(a.device))
    _lib.check(rc, "fsa_gate_merge_bwd")
    return d_a, d_b, d_c, d_gate
