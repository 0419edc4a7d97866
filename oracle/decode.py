"""CPU oracle for the one-step decode path (one new query per request).

TEST INFRASTRUCTURE ONLY - never imported by the product package.

Restates fsa_preview/ops/compressed_attention_decode.py and
fsa_preview/ops/selected_attention_decode.py of the reference, generalised from
the reference's batch of one to a batch of requests.

Two conventions are provided where the reference as written and the evident
intent differ:
  * block scores: `as_written=True` follows compressed_attention_decode.py:299
    (number of candidate blocks = ceil(compressed_len / B_K), the query's own
    block taken as 0) and :560,568 (kv head kh scores q-head kh); the default
    uses ceil(L / B_K) blocks, own block (L-1)//B_K and the first q-head of the
    group, i.e. what the prefill path computes for the last token.
  * selected attention: the reference calls the prefill kernel with a query of
    length 1, which reduces to O = v[0] (selected_attention_decode.py:29-40 with
    nsa_ref/ops/topk_sparse_attention.py:116-119,162); `as_written_selected_ref`
    gives that closed form, `decode_selected_attention_ref` the attention over
    the selected blocks of the cache.

Pinning status (tests/test_oracle_decode.py):
  decode_compressed_attention_ref : pinned - equals the last row of the prefill
      oracle (itself pinned against SDPA) on a consistent cache.
  decode_block_scores_ref / decode_topk_ref : pinned - default mode equals the
      prefill oracle's last row; as-written mode by brute-force loops.
  decode_selected_attention_ref : pinned - equals the prefill selected-attention
      oracle for the last token; softmax over an explicit key list.
"""
from __future__ import annotations

import math

import torch

LOG2E = 1.4426950408889634


def _bounds(cu):
    cu = [int(x) for x in cu]
    return [(cu[i], cu[i + 1]) for i in range(len(cu) - 1)]


def decode_compressed_attention_ref(q, ck, cv, cu_ck, pos, kernel_size, kernel_stride, softmax_scale=None,
                                    dtype=torch.float32):
    """q [B,Hq,D] (one query per request at position pos[b]); compressed key j of
    request b visible iff j*stride + ks - 1 <= pos[b].  Returns O [B,Hq,D] and
    base-2 LSE [Hq,B]; no visible key -> O = 0, LSE = -inf."""
    B, Hq, D = q.shape
    Hkv = ck.shape[1]
    g = Hq // Hkv
    if softmax_scale is None:
        softmax_scale = 1.0 / math.sqrt(D)
    c = softmax_scale * LOG2E
    o = torch.zeros(B, Hq, D, dtype=dtype)
    lse = torch.full((Hq, B), float("-inf"), dtype=dtype)
    for b, (k0, k1) in enumerate(_bounds(cu_ck)):
        nvis = min(k1 - k0, (int(pos[b]) - kernel_size + 1) // kernel_stride + 1) if int(pos[b]) >= kernel_size - 1 else 0
        if nvis <= 0:
            continue
        kx = ck[k0:k0 + nvis].to(dtype).repeat_interleave(g, dim=1)
        vx = cv[k0:k0 + nvis].to(dtype).repeat_interleave(g, dim=1)
        s = torch.einsum("hd,jhd->hj", q[b].to(dtype), kx) * c
        l2 = torch.logsumexp(s / LOG2E, -1) * LOG2E
        p = torch.exp2(s - l2[:, None])
        o[b] = torch.einsum("hj,jhd->hd", p, vx)
        lse[:, b] = l2
    return o, lse


def decode_block_scores_ref(q, ck, lse, cu_ck, pos, seqlens, kernel_size, kernel_stride, block_size,
                            init_blocks=1, local_blocks=2, softmax_scale=None, as_written=False,
                            nblk_cols=None):
    """fp32 [Hkv, B, nblk]: re-binned probabilities of one q-head per kv head plus
    forced (+inf) blocks; columns beyond a request's own block count are -inf so
    that they are never selected."""
    B, Hq, D = q.shape
    Hkv = ck.shape[1]
    g = Hq // Hkv
    if softmax_scale is None:
        softmax_scale = 1.0 / math.sqrt(D)
    c = softmax_scale * LOG2E
    na, ne = kernel_size // kernel_stride, block_size // kernel_stride
    w = [min(o, na + ne - 2 - o, na - 1, ne - 1) + 1 for o in range(na + ne - 1)]
    pad = na - 1
    kb = _bounds(cu_ck)
    nblks = []
    for b, (k0, k1) in enumerate(kb):
        nblks.append(math.ceil((k1 - k0) / block_size) if as_written else math.ceil(int(seqlens[b]) / block_size))
    ncol = nblk_cols if nblk_cols is not None else max(nblks + [1])
    out = torch.full((Hkv, B, ncol), float("-inf"), dtype=torch.float32)
    for b, (k0, k1) in enumerate(kb):
        nc = k1 - k0
        nvis = min(nc, (int(pos[b]) - kernel_size + 1) // kernel_stride + 1) if int(pos[b]) >= kernel_size - 1 else 0
        bq = 0 if as_written else (int(seqlens[b]) - 1) // block_size
        for kh in range(Hkv):
            hq = kh if as_written else kh * g
            prob = torch.zeros(max(nc, 1), dtype=torch.float32)
            if nvis > 0:
                s = (ck[k0:k0 + nvis, kh].float() @ q[b, hq].float()) * c
                prob[:nvis] = torch.exp2(s - lse[hq, b].float())
            for blk in range(nblks[b]):
                if blk < init_blocks or (bq >= blk and bq < blk + local_blocks):
                    out[kh, b, blk] = float("inf")
                    continue
                acc = 0.0
                for o_, wo in enumerate(w):
                    col = blk * ne - pad + o_
                    if 0 <= col < nvis:
                        acc += wo * float(prob[col])
                out[kh, b, blk] = acc
    return out


def decode_topk_ref(block_score, topk: int):
    """int32 [Hkv, B, topk]: ids by (score desc, id asc); slots for which no block is
    left (score -inf = beyond the request's blocks, or fewer columns than topk) are -1."""
    hkv, b, ncol = block_score.shape
    t = min(topk, ncol)
    order = torch.sort(block_score, dim=-1, descending=True, stable=True)
    idx = torch.full((hkv, b, topk), -1, dtype=torch.int32)
    sel = order.indices[..., :t].to(torch.int32)
    sel[order.values[..., :t] == float("-inf")] = -1
    idx[..., :t] = sel
    return idx


def decode_selected_attention_ref(q, k_cache, v_cache, cu_k, topk_idx, block_size, softmax_scale=None,
                                  dtype=torch.float32):
    """q [B,Hq,D]; k_cache/v_cache [total, Hkv, D] with cu_k [B+1] (the new token
    already appended); topk_idx [Hkv,B,T] block ids local to the request, entries
    < 0 or beyond the cache ignored, duplicates counted once.  Keys = every cached
    position of the selected blocks.  Returns O [B,Hq,D], base-2 LSE [Hq,B]."""
    B, Hq, D = q.shape
    Hkv = k_cache.shape[1]
    g = Hq // Hkv
    if softmax_scale is None:
        softmax_scale = 1.0 / math.sqrt(D)
    c = softmax_scale * LOG2E
    o = torch.zeros(B, Hq, D, dtype=dtype)
    lse = torch.full((Hq, B), float("-inf"), dtype=dtype)
    for b, (k0, k1) in enumerate(_bounds(cu_k)):
        L = k1 - k0
        for kh in range(Hkv):
            blocks = sorted({int(x) for x in topk_idx[kh, b] if 0 <= int(x) * block_size < L})
            if not blocks:
                continue
            keys = torch.cat([torch.arange(x * block_size, min(L, (x + 1) * block_size)) for x in blocks])
            kk = k_cache[k0 + keys, kh].to(dtype)
            vv = v_cache[k0 + keys, kh].to(dtype)
            hs = slice(kh * g, (kh + 1) * g)
            s = (q[b, hs].to(dtype) @ kk.t()) * c
            l2 = torch.logsumexp(s / LOG2E, -1) * LOG2E
            o[b, hs] = torch.exp2(s - l2[:, None]) @ vv
            lse[hs, b] = l2
    return o, lse


def as_written_selected_ref(q, k_cache, v_cache, cu_k, softmax_scale=None, dtype=torch.float32):
    """The reference's decode call as written: only key 0 of each request survives."""
    B, Hq, D = q.shape
    Hkv = k_cache.shape[1]
    g = Hq // Hkv
    if softmax_scale is None:
        softmax_scale = 1.0 / math.sqrt(D)
    o = torch.zeros(B, Hq, D, dtype=dtype)
    lse = torch.zeros(Hq, B, dtype=dtype)
    for b, (k0, _) in enumerate(_bounds(cu_k)):
        for h in range(Hq):
            o[b, h] = v_cache[k0, h // g].to(dtype)
            lse[h, b] = LOG2E * softmax_scale * float(q[b, h].to(dtype) @ k_cache[k0, h // g].to(dtype))
    return o, lse
