"""CPU oracle for compressed attention, block scores and top-k block selection.

TEST INFRASTRUCTURE ONLY - never imported by the product package.

Restates nsa_ref/ops/compressed_attention.py and nsa_ref/ops/linear_compress.py
of the reference in plain PyTorch on the CPU.

Pinning status (tests/test_oracle_cmpattn.py):
  linear_compress_ref      : pinned - brute-force loops; equals unfold + matmul.
  compressed_attention_ref : pinned - SDPA with an explicit bool mask, closed
      forms (first visible query sees exactly compressed key 0; queries before
      kernel_size-1 give O = 0, LSE = -inf), rows of P sum to 1.
  attention_score_ref      : pinned - equals softmax probabilities of the first
      head of each group; rows sum to 1 where any key is visible.
  transform_score_ref      : pinned - brute-force double loop over (offset, block)
      built from the reference's histogram construction of the weights.
  topk_select_ref          : pinned - torch.topk + sort on rows without a tie at
      the k-th value; tie rule (larger value first, then lower block id) is this
      build's own and is documented as such.
"""
from __future__ import annotations

import math
from typing import Optional, Tuple

import torch

LOG2E = 1.4426950408889634


def _bounds(cu) -> list:
    cu = [int(x) for x in cu]
    return [(cu[i], cu[i + 1]) for i in range(len(cu) - 1)]


def compressed_lens(cu_seqlens, kernel_size: int, kernel_stride: int):
    """y_len = floor((len - ks) / stride) + 1, 0 if len < ks (linear_compress.py:333-337)."""
    out = [0]
    for (s0, s1) in _bounds(cu_seqlens):
        L = s1 - s0
        out.append(out[-1] + ((L - kernel_size) // kernel_stride + 1 if L >= kernel_size else 0))
    return out


def linear_compress_ref(x: torch.Tensor, w: torch.Tensor, cu_seqlens, kernel_size: int, kernel_stride: int,
                        pe: Optional[torch.Tensor] = None, dtype=torch.float32):
    """y[n, h, :] = sum_k (x[n*stride + k, h, :] (+ pe[h, k, :])) @ W[h, k]  with W = w.view(H, ks, D, Dout)
    (linear_compress.py:28-131, 495-502: the positional term is added as
    einsum('h k d, h k d D -> h D', pe, W) to every compressed token)."""
    N, H, D = x.shape
    Dout = w.shape[-1]
    W = w.to(dtype).reshape(H, kernel_size, D, Dout)
    cu_y = compressed_lens(cu_seqlens, kernel_size, kernel_stride)
    ys = []
    for s, (s0, s1) in enumerate(_bounds(cu_seqlens)):
        ny = cu_y[s + 1] - cu_y[s]
        if ny == 0:
            continue
        xs = x[s0:s1].to(dtype)
        win = xs.unfold(0, kernel_size, kernel_stride)[:ny]  # [ny, H, D, ks]
        ys.append(torch.einsum("nhdk,hkde->nhe", win, W))
    y = torch.cat(ys, 0) if ys else x.new_zeros((0, H, Dout), dtype=dtype)
    if pe is not None:
        y = y + torch.einsum("hkd,hkde->he", pe.to(dtype), W)[None]
    return y, cu_y


def visible_mask(Lq: int, Nc: int, kernel_size: int, kernel_stride: int) -> torch.Tensor:
    """[Lq, Nc] bool: compressed key j visible to query i iff i >= j*stride + ks - 1
    (compressed_attention.py:110,123)."""
    i = torch.arange(Lq)[:, None]
    j = torch.arange(Nc)[None, :]
    return i >= j * kernel_stride + kernel_size - 1


def compressed_attention_ref(q, ck, cv, kernel_size, kernel_stride, cu_seqlens_q, cu_seqlens_k,
                             softmax_scale=None, dtype=torch.float32):
    """(O [N,Hq,D], LSE2 [Hq,N]); queries with no visible key: O = 0, LSE2 = -inf
    (compressed_attention.py:27-156, 547-553).  Differentiable."""
    N, Hq, D = q.shape
    Hkv = ck.shape[1]
    g = Hq // Hkv
    if softmax_scale is None:
        softmax_scale = 1.0 / math.sqrt(D)
    c = softmax_scale * LOG2E
    o = []
    lse = []
    for (q0, q1), (k0, k1) in zip(_bounds(cu_seqlens_q), _bounds(cu_seqlens_k)):
        Lq, Nc = q1 - q0, k1 - k0
        qs = q[q0:q1].to(dtype)
        if Nc == 0:
            o.append(torch.zeros(Lq, Hq, D, dtype=dtype))
            lse.append(torch.full((Hq, Lq), float("-inf"), dtype=dtype))
            continue
        kx = ck[k0:k1].to(dtype).repeat_interleave(g, dim=1)
        vx = cv[k0:k1].to(dtype).repeat_interleave(g, dim=1)
        vis = visible_mask(Lq, Nc, kernel_size, kernel_stride)
        s = torch.einsum("ihd,jhd->hij", qs, kx) * c
        s = s.masked_fill(~vis[None], float("-inf"))
        m = s.max(-1, keepdim=True).values
        m = torch.where(torch.isinf(m), torch.zeros_like(m), m)
        p = torch.exp2(s - m)
        l = p.sum(-1, keepdim=True)
        any_vis = vis.any(-1)[None, :, None]
        pn = torch.where(any_vis, p / l.clamp_min(1e-300 if dtype == torch.float64 else 1e-38), torch.zeros_like(p))
        o.append(torch.einsum("hij,jhd->ihd", pn, vx))
        ls = (m + torch.log2(l)).squeeze(-1)
        lse.append(torch.where(vis.any(-1)[None], ls, torch.full_like(ls, float("-inf"))))
    return torch.cat(o, 0), torch.cat(lse, 1)


def compressed_attention_grads_ref(q, ck, cv, kernel_size, kernel_stride, cu_seqlens_q, cu_seqlens_k, do,
                                   softmax_scale=None, dtype=torch.float32, round_dtype=None, o_in=None, lse_in=None):
    """(O, LSE2, dQ, dCK, dCV).  Without round_dtype: autograd through
    compressed_attention_ref.  With round_dtype (bf16 / fp16): the explicit
    formulas with the reference kernels' rounding points - P is cast to the
    input dtype before P^T dO and dS before dS K and dS^T Q
    (compressed_attention.py:336-352, 490-503) - accumulation in `dtype`.
    o_in / lse_in: the saved forward output and LSE the backward operator takes
    as inputs (compressed_attention.py:600-640); used for delta and P when given."""
    if round_dtype is None and o_in is None and lse_in is None:
        q_, k_, v_ = (x.detach().to(dtype).requires_grad_(True) for x in (q, ck, cv))
        o, lse = compressed_attention_ref(q_, k_, v_, kernel_size, kernel_stride, cu_seqlens_q, cu_seqlens_k,
                                          softmax_scale, dtype)
        (o * do.to(dtype)).sum().backward()
        return o.detach(), lse.detach(), q_.grad, k_.grad, v_.grad
    N, Hq, D = q.shape
    Hkv = ck.shape[1]
    g = Hq // Hkv
    if softmax_scale is None:
        softmax_scale = 1.0 / math.sqrt(D)
    c = softmax_scale * LOG2E
    o, lse = compressed_attention_ref(q, ck, cv, kernel_size, kernel_stride, cu_seqlens_q, cu_seqlens_k,
                                      softmax_scale, dtype)
    qf, kf, vf, dof = (x.detach().to(dtype) for x in (q, ck, cv, do))
    dq = torch.zeros_like(qf)
    dk = torch.zeros_like(kf)
    dv = torch.zeros_like(vf)

    def rnd(x):
        return x if round_dtype is None else x.to(round_dtype).to(dtype)

    o_use = o if o_in is None else o_in.to(dtype)
    lse_use = lse if lse_in is None else lse_in.to(dtype)
    for (q0, q1), (k0, k1) in zip(_bounds(cu_seqlens_q), _bounds(cu_seqlens_k)):
        Lq, Nc = q1 - q0, k1 - k0
        if Nc == 0 or Lq == 0:
            continue
        vis = visible_mask(Lq, Nc, kernel_size, kernel_stride)
        for h in range(Hq):
            kh = h // g
            s = (qf[q0:q1, h] @ kf[k0:k1, kh].t()) * c
            ls = lse_use[h, q0:q1, None]
            p = torch.where(vis, torch.exp2(s - torch.where(torch.isinf(ls), torch.zeros_like(ls), ls)),
                            torch.zeros_like(s))
            dp = dof[q0:q1, h] @ vf[k0:k1, kh].t()
            delta = (o_use[q0:q1, h] * dof[q0:q1, h]).sum(-1, keepdim=True)
            ds = rnd(softmax_scale * p * (dp - delta))
            dq[q0:q1, h] = ds @ kf[k0:k1, kh]
            dk[k0:k1, kh] += ds.t() @ qf[q0:q1, h]
            dv[k0:k1, kh] += rnd(p).t() @ dof[q0:q1, h]
    return o, lse, dq, dk, dv


def attention_score_ref(q, ck, lse, kernel_size, kernel_stride, cu_seqlens_q, cu_seqlens_k, softmax_scale=None,
                        dtype=torch.float32):
    """score[kh, i, j] = 2^(c q[i, kh*g] . ck[j, kh] - lse[kh*g, i]) if visible else 0, fp32
    [Hkv, N, max_k].  Only the FIRST q-head of each group is used
    (compressed_attention.py:893-920 with the per-head slicing of :1280-1283)."""
    N, Hq, D = q.shape
    Hkv = ck.shape[1]
    g = Hq // Hkv
    if softmax_scale is None:
        softmax_scale = 1.0 / math.sqrt(D)
    c = softmax_scale * LOG2E
    kb = _bounds(cu_seqlens_k)
    max_k = max(k1 - k0 for (k0, k1) in kb)
    score = torch.zeros(Hkv, N, max_k, dtype=dtype)
    for (q0, q1), (k0, k1) in zip(_bounds(cu_seqlens_q), kb):
        Lq, Nc = q1 - q0, k1 - k0
        if Nc == 0:
            continue
        q0h = q[q0:q1, ::g].to(dtype)  # first head of each group: [Lq, Hkv, D]
        s = torch.einsum("ihd,jhd->hij", q0h, ck[k0:k1].to(dtype)) * c
        vis = visible_mask(Lq, Nc, kernel_size, kernel_stride)
        pr = torch.exp2(s - lse[::g, q0:q1].to(dtype)[:, :, None])
        score[:, q0:q1, :Nc] = torch.where(vis[None], pr, torch.zeros_like(pr))
    return score


def score_weights(kernel_size: int, kernel_stride: int, block_size: int) -> torch.Tensor:
    """w[o] = #{(a, e): a < ks/stride, e < B_K/stride, a + e = o} (compressed_attention.py:1110-1115)."""
    na, ne = kernel_size // kernel_stride, block_size // kernel_stride
    w = torch.zeros(na + ne - 1)
    for a in range(na):
        for e in range(ne):
            w[a + e] += 1
    return w


def transform_score_ref(score, kernel_size, kernel_stride, block_size, cu_seqlens_q, max_seqlen_q=None,
                        init_blocks: int = 1, local_blocks: int = 2):
    """block_score[kh, i, b] = sum_o w[o] * score[kh, i, b*(B_K/stride) - (ks/stride - 1) + o]
    (out-of-range columns count as 0), then +inf where b < init_blocks or
    i//B_K - local_blocks < b <= i//B_K (compressed_attention.py:1046-1084, 1099-1115)."""
    Hkv, N, max_k = score.shape
    qb = _bounds(cu_seqlens_q)
    if max_seqlen_q is None:
        max_seqlen_q = max(q1 - q0 for (q0, q1) in qb)
    nblk = (max_seqlen_q + block_size - 1) // block_size
    w = score_weights(kernel_size, kernel_stride, block_size).to(score.dtype)
    pad = kernel_size // kernel_stride - 1
    bs = block_size // kernel_stride
    out = torch.zeros(Hkv, N, nblk, dtype=score.dtype)
    cols = torch.arange(nblk) * bs - pad
    for o_ in range(w.numel()):
        c = cols + o_
        ok = (c >= 0) & (c < max_k)
        out[:, :, ok] += w[o_] * score[:, :, c[ok]]
    for (q0, q1) in qb:
        bq = (torch.arange(q1 - q0) // block_size)[:, None]
        b = torch.arange(nblk)[None, :]
        force = (b < init_blocks) | ((bq >= b) & (bq < b + local_blocks))
        out[:, q0:q1] = torch.where(force[None], torch.full_like(out[:, q0:q1], float("inf")), out[:, q0:q1])
    return out


def topk_select_ref(block_score, topk: int, cu_seqlens_q, block_size: int, to_bf16: bool = True):
    """int32 [Hkv, N, min(T, nblk)]: ids of the T largest block scores (after the
    cast to bf16 the non-parallel path applies, compressed_attention.py:1306-1313),
    ascending, ids above the query's own block replaced by -1.
    Tie rule of this build: larger value first, then lower block id
    (torch.topk leaves the order of equal values unspecified)."""
    Hkv, N, nblk = block_score.shape
    t = min(topk, nblk)
    sc = block_score.to(torch.bfloat16).float() if to_bf16 else block_score.float()
    # stable sort by descending value keeps the lower index first among equals
    order = torch.sort(sc, dim=-1, descending=True, stable=True).indices[..., :t]
    idx = order.sort(-1).values
    for (q0, q1) in _bounds(cu_seqlens_q):
        bq = (torch.arange(q1 - q0) // block_size)[None, :, None]
        seg = idx[:, q0:q1]
        idx[:, q0:q1] = torch.where(seg > bq, torch.full_like(seg, -1), seg)
    return idx.to(torch.int32)


def kth_value_tie_rows(block_score, topk: int, to_bf16: bool = True) -> torch.Tensor:
    """bool [Hkv, N]: rows where the k-th and (k+1)-th largest scores are equal,
    i.e. where the selected SET depends on the tie rule."""
    nblk = block_score.shape[-1]
    t = min(topk, nblk)
    if t >= nblk:
        return torch.zeros(block_score.shape[:2], dtype=torch.bool)
    sc = block_score.to(torch.bfloat16).float() if to_bf16 else block_score.float()
    s = torch.sort(sc, dim=-1, descending=True).values
    return s[..., t - 1] == s[..., t]


def compressed_topk_ref(q, ck, lse, kernel_size, kernel_stride, block_size, topk, cu_seqlens_q, cu_seqlens_k,
                        softmax_scale=None, init_blocks=1, local_blocks=2, max_seqlen_q=None, to_bf16=True):
    score = attention_score_ref(q, ck, lse, kernel_size, kernel_stride, cu_seqlens_q, cu_seqlens_k, softmax_scale)
    bscore = transform_score_ref(score, kernel_size, kernel_stride, block_size, cu_seqlens_q, max_seqlen_q,
                                 init_blocks, local_blocks)
    return topk_select_ref(bscore, topk, cu_seqlens_q, block_size, to_bf16), bscore
