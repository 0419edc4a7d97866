"""CPU oracle for NSA *selected attention* and its inverted index.

TEST INFRASTRUCTURE ONLY - never imported by the product package.

Restates, in plain PyTorch/numpy on the CPU, what the reference computes in
  fsa/ops/FSA_topk_sparse_attention.py   (FSA kernels, index lists)
  nsa_ref/ops/topk_sparse_attention.py   (per-query semantics)

Pinning status (tests/test_oracle_selattn.py):
  selected_attention_ref : pinned - dense-mask fp64 softmax, SDPA with an
      explicit bool mask, closed forms (token 0, all-blocks == causal,
      own-block only == block-diagonal causal), slot-permutation invariance.
  selected_attention_grads_ref : pinned - explicit backward formulas checked
      against autograd of the dense fp64 formulation, autograd of
      selected_attention_ref and central finite differences on tiny inputs.
  selected_attention_rows_ref : pinned - equals the two functions above on
      every row / block of small inputs (independent code path).
  key_block_grads_ref : pinned - equals selected_attention_rows_ref
      (key_block=...) summed over every query that selected the block, on small
      inputs, and the dK / dV slices of selected_attention_grads_ref.
  build_index_ref : pinned - brute-force Python loops, torch.bincount,
      exclusive cumsum identity.
"""
from __future__ import annotations

import math
from typing import Optional, Tuple

import numpy as np
import torch

LOG2E = 1.4426950408889634


def _seq_bounds(cu_seqlens) -> list:
    cu = [int(x) for x in cu_seqlens]
    return [(cu[i], cu[i + 1]) for i in range(len(cu) - 1)]


def selected_attention_ref(
    q: torch.Tensor,  # [N, Hq, D]
    k: torch.Tensor,  # [N, Hkv, D]
    v: torch.Tensor,  # [N, Hkv, D]
    topk_idx: torch.Tensor,  # [Hkv, N, T] int, -1 = padding, block ids local to the sequence
    block_size: int,
    cu_seqlens,
    softmax_scale: Optional[float] = None,
    q_chunk: int = 128,
    dtype: torch.dtype = torch.float32,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """O[N,Hq,D] and base-2 LSE[Hq,N].

    Per query i (sequence-local position) and q-head h with kv-head kh = h // g:
    key set = { p : p // B_K in topk_idx[kh, i, :], p <= i, p < len }
    (nsa_ref/ops/topk_sparse_attention.py:116-119,162;
     fsa/ops/FSA_topk_sparse_attention.py:520),
    s_p = scale * log2(e) * q.k  (FSA_topk_sparse_attention.py:318,523),
    LSE2 = log2 sum 2^s_p  (FSA_topk_sparse_attention.py:256-261,273),
    O = sum 2^(s_p - LSE2) v_p.
    Differentiable (autograd) in q, k, v.
    """
    N, Hq, D = q.shape
    Hkv = k.shape[1]
    g = Hq // Hkv
    T = topk_idx.shape[-1]
    if softmax_scale is None:
        softmax_scale = 1.0 / math.sqrt(D)
    c = softmax_scale * LOG2E
    qf, kf, vf = q.to(dtype), k.to(dtype), v.to(dtype)
    o_chunks = []
    lse_chunks = []
    ar = torch.arange(block_size)
    B = block_size
    for (s0, s1) in _seq_bounds(cu_seqlens):
        L = s1 - s0
        nblk = (L + B - 1) // B
        pad = nblk * B - L
        # [Hkv, nblk, B*D] block views of this sequence's keys / values (zero padded tail)
        kb = torch.nn.functional.pad(kf[s0:s1], (0, 0, 0, 0, 0, pad)).reshape(nblk, B, Hkv, D).permute(2, 0, 1, 3).reshape(Hkv, nblk, B * D)
        vb = torch.nn.functional.pad(vf[s0:s1], (0, 0, 0, 0, 0, pad)).reshape(nblk, B, Hkv, D).permute(2, 0, 1, 3).reshape(Hkv, nblk, B * D)
        for i0 in range(0, L, q_chunk):
            i1 = min(L, i0 + q_chunk)
            C = i1 - i0
            idx = topk_idx[:, s0 + i0 : s0 + i1, :].long()  # [Hkv, C, T]
            kpos = idx[..., None] * B + ar  # [Hkv, C, T, B]
            qpos = torch.arange(i0, i1)[None, :, None, None]
            valid = ((idx[..., None] >= 0) & (idx[..., None] < nblk) & (kpos <= qpos) & (kpos < L))
            valid = valid.reshape(Hkv, C, T * B)
            bsel = idx.clamp(0, nblk - 1).reshape(Hkv, C * T)
            qc = qf[s0 + i0 : s0 + i1].reshape(C, Hkv, g, D)
            o_h, lse_h = [], []
            for kh in range(Hkv):
                kg = kb[kh].index_select(0, bsel[kh]).reshape(C, T * B, D)
                vg = vb[kh].index_select(0, bsel[kh]).reshape(C, T * B, D)
                s = torch.bmm(qc[:, kh], kg.transpose(1, 2)) * c  # [C, g, TB]
                s = s.masked_fill(~valid[kh][:, None, :], float("-inf"))
                m = s.max(dim=-1, keepdim=True).values
                m = torch.where(torch.isinf(m), torch.zeros_like(m), m)
                p = torch.exp2(s - m)
                l = p.sum(-1, keepdim=True)
                lse_h.append((m + torch.log2(l)).squeeze(-1))  # [C, g]
                o_h.append(torch.bmm(p / l, vg))  # [C, g, D]
            o_chunks.append(torch.stack(o_h, 1).reshape(C, Hq, D))
            lse_chunks.append(torch.stack(lse_h, 1).reshape(C, Hq).t())
    return torch.cat(o_chunks, 0), torch.cat(lse_chunks, 1)


def selected_attention_grads_ref(q, k, v, topk_idx, block_size, cu_seqlens, do, softmax_scale=None,
                                 dtype=torch.float32, q_chunk: int = 128, round_dtype=None,
                                 o_in=None, lse_in=None):
    """(O, LSE2, dQ, dK, dV) by the explicit backward formulas, chunk by chunk.

    FSA_topk_sparse_attention.py:1229-1237 and :1697-1709 with P = 2^(s - LSE2):
    delta = sum_d O dO, dP = dO V^T, dS = scale * P * (dP - delta), dQ = dS K,
    dK = sum over the group's heads of dS^T Q, dV = sum over heads of P^T dO
    (dK/dV head sum: :1854-1855).  No autograd, so memory stays bounded; the
    formulas themselves are checked against autograd of the dense formulation
    and finite differences in the tests.

    o_in / lse_in: the backward operator of the reference takes the saved forward
    output and LSE as INPUTS (FSA_topk_sparse_attention.py:1715-1730: delta is
    computed from the stored, dtype-rounded O and P from the stored LSE); when
    given they are used in place of the recomputed ones, which is the functional
    specification of the backward op.

    round_dtype (bf16 / fp16) reproduces the reference kernels' rounding points:
    P is cast to the input dtype before P^T dO and dS before dS K and dS^T Q
    (FSA_topk_sparse_attention.py:1236, 1705-1706); accumulation stays in `dtype`.
    """
    def rnd(x):
        return x if round_dtype is None else x.to(round_dtype).to(dtype)

    N, Hq, D = q.shape
    Hkv = k.shape[1]
    g = Hq // Hkv
    T = topk_idx.shape[-1]
    B = block_size
    if softmax_scale is None:
        softmax_scale = 1.0 / math.sqrt(D)
    c = softmax_scale * LOG2E
    qf, kf, vf, dof = (x.detach().to(dtype) for x in (q, k, v, do))
    o_out = torch.empty_like(qf)
    lse_out = torch.empty(Hq, N, dtype=dtype)
    dq = torch.empty_like(qf)
    dk = torch.zeros_like(kf)
    dv = torch.zeros_like(vf)
    ar = torch.arange(B)
    for (s0, s1) in _seq_bounds(cu_seqlens):
        L = s1 - s0
        if L == 0:
            continue
        nblk = (L + B - 1) // B
        pad = nblk * B - L
        kb = torch.nn.functional.pad(kf[s0:s1], (0, 0, 0, 0, 0, pad)).reshape(nblk, B, Hkv, D).permute(2, 0, 1, 3).reshape(Hkv, nblk, B * D)
        vb = torch.nn.functional.pad(vf[s0:s1], (0, 0, 0, 0, 0, pad)).reshape(nblk, B, Hkv, D).permute(2, 0, 1, 3).reshape(Hkv, nblk, B * D)
        dkb = torch.zeros_like(kb)
        dvb = torch.zeros_like(vb)
        for i0 in range(0, L, q_chunk):
            i1 = min(L, i0 + q_chunk)
            C = i1 - i0
            idx = topk_idx[:, s0 + i0 : s0 + i1, :].long()
            kpos = idx[..., None] * B + ar
            qpos = torch.arange(i0, i1)[None, :, None, None]
            valid = ((idx[..., None] >= 0) & (idx[..., None] < nblk) & (kpos <= qpos) & (kpos < L))
            valid = valid.reshape(Hkv, C, T * B)
            bsel = idx.clamp(0, nblk - 1).reshape(Hkv, C * T)
            qc = qf[s0 + i0 : s0 + i1].reshape(C, Hkv, g, D)
            doc = dof[s0 + i0 : s0 + i1].reshape(C, Hkv, g, D)
            for kh in range(Hkv):
                kg = kb[kh].index_select(0, bsel[kh]).reshape(C, T * B, D)
                vg = vb[kh].index_select(0, bsel[kh]).reshape(C, T * B, D)
                s = torch.bmm(qc[:, kh], kg.transpose(1, 2)) * c
                s = s.masked_fill(~valid[kh][:, None, :], float("-inf"))
                lse = torch.logsumexp(s * (1.0 / LOG2E), dim=-1, keepdim=True) * LOG2E  # base 2
                hs = slice(kh * g, (kh + 1) * g)
                o = torch.bmm(torch.exp2(s - lse), vg)
                lse_use = lse if lse_in is None else lse_in[hs, s0 + i0 : s0 + i1].to(dtype).t()[:, :, None]
                o_use = o if o_in is None else o_in[s0 + i0 : s0 + i1, hs].to(dtype)
                p = torch.exp2(s - lse_use)
                dp = torch.bmm(doc[:, kh], vg.transpose(1, 2))
                delta = (o_use * doc[:, kh]).sum(-1, keepdim=True)
                ds = softmax_scale * p * (dp - delta)
                o_out[s0 + i0 : s0 + i1, hs] = o
                lse_out[hs, s0 + i0 : s0 + i1] = lse.squeeze(-1).t()
                ds_c, p_c = rnd(ds), rnd(p)
                dq[s0 + i0 : s0 + i1, hs] = torch.bmm(ds_c, kg)
                dkb[kh].index_add_(0, bsel[kh], torch.bmm(ds_c.transpose(1, 2), qc[:, kh]).reshape(C * T, B * D))
                dvb[kh].index_add_(0, bsel[kh], torch.bmm(p_c.transpose(1, 2), doc[:, kh]).reshape(C * T, B * D))
        dk[s0:s1] = dkb.reshape(Hkv, nblk * B, D)[:, :L].permute(1, 0, 2)
        dv[s0:s1] = dvb.reshape(Hkv, nblk * B, D)[:, :L].permute(1, 0, 2)
    return o_out, lse_out, dq, dk, dv


def selected_attention_rows_ref(q, k, v, topk_idx, block_size, cu_seqlens, rows, do=None, softmax_scale=None,
                                o_in=None, lse_in=None, round_dtype=None, key_block=None, dtype=torch.float64):
    """The same quantities for a SAMPLE of queries, one explicit key list per (row, kv head).

    rows: global query rows.  Returns dict with o [R,Hq,D], lse [Hq,R] (base 2) and, if `do` is given, dq [R,Hq,D]
    plus - when key_block = (kv head, global first row of the block) - the sum over the sampled rows and the group's
    heads of their contributions to dK and dV of that block's keys (dk_block, dv_block [B_K, D], rows beyond the
    sequence end zero).  Written independently of the chunked functions above (no block views, no batched gathers)
    so that either can check the other; same formulas and rounding points (see selected_attention_grads_ref)."""
    def rnd(x):
        return x if round_dtype is None else x.to(round_dtype).to(dtype)

    N, Hq, D = q.shape
    Hkv = k.shape[1]
    g = Hq // Hkv
    B = block_size
    if softmax_scale is None:
        softmax_scale = 1.0 / math.sqrt(D)
    c = softmax_scale * LOG2E
    bounds = _seq_bounds(cu_seqlens)
    starts = np.array([b[0] for b in bounds])
    R = len(rows)
    out = {"o": torch.zeros(R, Hq, D, dtype=dtype), "lse": torch.full((Hq, R), float("-inf"), dtype=dtype)}
    if do is not None:
        out["dq"] = torch.zeros(R, Hq, D, dtype=dtype)
        if key_block is not None:
            out["dk_block"] = torch.zeros(B, D, dtype=dtype)
            out["dv_block"] = torch.zeros(B, D, dtype=dtype)
    for r, row in enumerate(int(x) for x in rows):
        si = int(np.searchsorted(starts, row, side="right")) - 1
        s0, s1 = bounds[si]
        i, L = row - s0, s1 - s0
        for kh in range(Hkv):
            blocks = sorted({int(x) for x in topk_idx[kh, row] if int(x) >= 0 and int(x) * B <= i})
            if not blocks:
                continue
            keys = torch.cat([torch.arange(x * B, min((x + 1) * B, i + 1, L)) for x in blocks]) + s0
            kk, vv = k[keys, kh].to(dtype), v[keys, kh].to(dtype)
            hs = slice(kh * g, (kh + 1) * g)
            sc = (q[row, hs].to(dtype) @ kk.t()) * c                      # [g, nkeys]
            lse = torch.logsumexp(sc / LOG2E, -1) * LOG2E
            o = torch.exp2(sc - lse[:, None]) @ vv
            out["o"][r, hs], out["lse"][hs, r] = o, lse
            if do is None:
                continue
            lse_use = lse if lse_in is None else lse_in[hs, row].to(dtype)
            o_use = o if o_in is None else o_in[row, hs].to(dtype)
            dor = do[row, hs].to(dtype)
            p = torch.exp2(sc - lse_use[:, None])
            ds = softmax_scale * p * (dor @ vv.t() - (o_use * dor).sum(-1, keepdim=True))
            ds_c, p_c = rnd(ds), rnd(p)
            out["dq"][r, hs] = ds_c @ kk
            if key_block is not None and key_block[0] == kh:
                inblk = (keys >= key_block[1]) & (keys < key_block[1] + B)
                if bool(inblk.any()):
                    off = keys[inblk] - key_block[1]
                    out["dk_block"][off] += ds_c[:, inblk].t() @ q[row, hs].to(dtype)
                    out["dv_block"][off] += p_c[:, inblk].t() @ dor
    return out


def key_block_grads_ref(q, k, v, do, o_in, lse_in, kv_head: int, block_row0: int, users, block_size: int,
                        seq_end: int, softmax_scale=None, round_dtype=None, dtype=torch.float64, chunk: int = 8192):
    """dK, dV [B_K, D] of ONE key block (kv head `kv_head`, first global row `block_row0`) from ALL the queries
    in `users` (global rows of the queries that selected the block), vectorised so that a block selected by every
    query of a 64K sequence is cheap.  The backward operator takes the stored forward output and LSE as inputs
    (FSA_topk_sparse_attention.py:1715-1730), so o_in [N, Hq, D] and lse_in [Hq, N] (base 2) are required:
    P = 2^(c q.k - LSE2) for key row <= query row (:520), delta = sum_d O dO, dS = scale * P * (dO.v - delta),
    dK = sum dS^T q, dV = sum P^T dO over the users and the g heads of the group (:1697-1709, 1854-1855), with P
    and dS cast to round_dtype before the second products when given (:1705-1706).  Rows of the block at or past
    seq_end are zero."""
    def rnd(x):
        return x if round_dtype is None else x.to(round_dtype).to(dtype)

    N, Hq, D = q.shape
    g = Hq // k.shape[1]
    B = block_size
    if softmax_scale is None:
        softmax_scale = 1.0 / math.sqrt(D)
    c = softmax_scale * LOG2E
    nk = min(B, seq_end - block_row0)
    kk = k[block_row0 : block_row0 + nk, kv_head].to(dtype)          # [nk, D]
    vv = v[block_row0 : block_row0 + nk, kv_head].to(dtype)
    hs = slice(kv_head * g, (kv_head + 1) * g)
    users = torch.as_tensor(users, dtype=torch.long)
    dk = torch.zeros(B, D, dtype=dtype)
    dv = torch.zeros(B, D, dtype=dtype)
    key_rows = block_row0 + torch.arange(nk)
    for u0 in range(0, users.numel(), chunk):
        u = users[u0 : u0 + chunk]
        qr, dor, orr = (x[u][:, hs].to(dtype) for x in (q, do, o_in))   # [C, g, D]
        lse = lse_in[hs][:, u].to(dtype).t()[:, :, None]                # [C, g, 1]
        sc = torch.einsum("cgd,kd->cgk", qr, kk) * c
        vis = (key_rows[None, :] <= u[:, None])[:, None, :]             # [C, 1, nk]
        p = torch.where(vis, torch.exp2(sc - lse), torch.zeros((), dtype=dtype))
        dp = torch.einsum("cgd,kd->cgk", dor, vv)
        delta = (orr * dor).sum(-1, keepdim=True)
        ds = softmax_scale * p * (dp - delta)
        ds_c, p_c = rnd(ds), rnd(p)
        dk[:nk] += torch.einsum("cgk,cgd->kd", ds_c, qr)
        dv[:nk] += torch.einsum("cgk,cgd->kd", p_c, dor)
    return dk, dv


def dense_mask(topk_idx: torch.Tensor, block_size: int, cu_seqlens) -> torch.Tensor:
    """Bool [Hkv, N, N]: mask[kh, i, p] = key p (global row) visible to query i."""
    Hkv, N, T = topk_idx.shape
    mask = torch.zeros(Hkv, N, N, dtype=torch.bool)
    for (s0, s1) in _seq_bounds(cu_seqlens):
        L = s1 - s0
        pos = torch.arange(L)
        blk = pos // block_size
        for kh in range(Hkv):
            idx = topk_idx[kh, s0:s1].long()  # [L, T]
            sel = (idx[:, :, None] == blk[None, None, :]).any(1)  # [L(query), L(key)]
            sel &= pos[None, :] <= pos[:, None]
            mask[kh, s0:s1, s0:s1] = sel
    return mask


def selected_attention_dense_ref(q, k, v, topk_idx, block_size, cu_seqlens, softmax_scale=None,
                                 dtype=torch.float64):
    """Same quantity via an explicit [N, N] mask and torch.softmax (small N only)."""
    N, Hq, D = q.shape
    Hkv = k.shape[1]
    g = Hq // Hkv
    if softmax_scale is None:
        softmax_scale = 1.0 / math.sqrt(D)
    mask = dense_mask(topk_idx, block_size, cu_seqlens)  # [Hkv, N, N]
    qf, kf, vf = q.to(dtype), k.to(dtype), v.to(dtype)
    kx = kf.repeat_interleave(g, dim=1)
    vx = vf.repeat_interleave(g, dim=1)
    mx = mask.repeat_interleave(g, dim=0)  # [Hq, N, N]
    s = torch.einsum("ihd,phd->hip", qf, kx) * softmax_scale
    s = s.masked_fill(~mx, float("-inf"))
    p = torch.softmax(s, dim=-1)
    o = torch.einsum("hip,phd->ihd", p, vx)
    lse2 = torch.logsumexp(s, dim=-1) * LOG2E
    return o, lse2


def build_index_ref(topk_idx: torch.Tensor, cu_seqlens, block_size: int):
    """Inverted block->query index, all sequences at once, global numbering.

    Block b of sequence s has global id cu_blocks[s] + b with
    cu_blocks = cumsum(ceil(len_s / B_K)).  Per kv head:
      counts[gb]      = number of (query, slot) entries naming that block
                        (torch.bincount, FSA_topk_sparse_attention.py:951-955)
      starts          = exclusive cumsum of counts (:1018), length NB + 1
      sel_tokens[p]   = query ids (global rows) grouped by block, ascending
                        inside a block (row-major compaction of a
                        [nblk, N] table, :1016)
      slot_of[i, t]   = position p of entry (i, t) in sel_tokens, -1 for
                        padding; slot_of - starts[gb] is the reference's
                        token_index_mapping (:641-649)
    Entries that are negative or name a block past the sequence end are
    ignored.  Returns numpy int32 arrays (cu_blocks, counts, starts,
    sel_tokens[Hkv, N*T] (-1 tail), slot_of[Hkv, N, T]).
    """
    t = topk_idx.cpu().numpy().astype(np.int64)
    Hkv, N, T = t.shape
    bounds = _seq_bounds(cu_seqlens)
    nblk = [(s1 - s0 + block_size - 1) // block_size for (s0, s1) in bounds]
    cu_blocks = np.zeros(len(bounds) + 1, dtype=np.int64)
    cu_blocks[1:] = np.cumsum(nblk)
    NB = int(cu_blocks[-1])
    gkey = np.full((Hkv, N, T), NB, dtype=np.int64)
    for s, (s0, s1) in enumerate(bounds):
        loc = t[:, s0:s1, :]
        ok = (loc >= 0) & (loc < nblk[s])
        gkey[:, s0:s1, :] = np.where(ok, loc + cu_blocks[s], NB)
    counts = np.zeros((Hkv, NB), dtype=np.int32)
    starts = np.zeros((Hkv, NB + 1), dtype=np.int32)
    sel_tokens = np.full((Hkv, N * T), -1, dtype=np.int32)
    slot_of = np.full((Hkv, N, T), -1, dtype=np.int32)
    for h in range(Hkv):
        flat = gkey[h].reshape(-1)
        order = np.argsort(flat, kind="stable")
        skeys = flat[order]
        nvalid = int((skeys < NB).sum())
        counts[h] = np.bincount(skeys[:nvalid], minlength=NB)[:NB]
        starts[h, 1:] = np.cumsum(counts[h])
        sel_tokens[h, :nvalid] = (order[:nvalid] // T).astype(np.int32)
        so = slot_of[h].reshape(-1)
        so[order[:nvalid]] = np.arange(nvalid, dtype=np.int32)
    return cu_blocks.astype(np.int32), counts, starts, sel_tokens, slot_of


def count_pairs(topk_idx: torch.Tensor, block_size: int, cu_seqlens) -> Tuple[int, int]:
    """(valid (query, block) pairs summed over kv heads,
        unmasked (query, key) pairs summed over kv heads)."""
    Hkv, N, T = topk_idx.shape
    pairs = 0
    keys = 0
    for (s0, s1) in _seq_bounds(cu_seqlens):
        L = s1 - s0
        idx = topk_idx[:, s0:s1].long()
        pos = torch.arange(L)[None, :, None]
        nb = (L + block_size - 1) // block_size
        ok = (idx >= 0) & (idx < nb)
        lo = idx * block_size
        n = (torch.minimum(pos, lo + block_size - 1) - lo + 1).clamp(min=0)
        n = torch.where(ok, n, torch.zeros_like(n))
        pairs += int(ok.sum())
        keys += int(n.sum())
    return pairs, keys
