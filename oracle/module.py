"""CPU oracle for the pieces around the hot path that the module needs:
sliding-window attention, rotary embedding, the gated sum, the whole layer.

TEST INFRASTRUCTURE ONLY - never imported by the product package.

Restates fsa/module/fsa.py and nsa_ref/module/rope.py of the reference.  Two
third-party routines the reference calls are not part of it and are restated
from their published definitions:
  * flash_attn.flash_attn_varlen_func(causal=True, window_size=(W, -1)):
    the query at position i attends keys p with i - W <= p <= i;
  * flash_attn.layers.rotary.apply_rotary_emb (non-interleaved): with
    x = [x1 | x2] split at D/2, out = [x1 cos - x2 sin | x1 sin + x2 cos];
  * transformers ROPE_INIT_FUNCTIONS["llama3"] (frequency table).

Pinning status (tests/test_oracle_module.py):
  window_attention_ref : pinned - SDPA with an explicit band mask; window >= length
      equals causal attention.
  llama3_inv_freq      : pinned - against transformers' own function (importable here);
      factor 1 reduces to 1 / theta^(2i/D).
  rope_ref             : pinned - norm preservation, relative-position property of the
      rotated dot product, position 0 is the identity.
  fsa_layer_ref        : composition of pinned pieces (no independent pin beyond shape
      and gradient flow) - the layer-level GPU test therefore compares like for like.
"""
from __future__ import annotations

import math

import torch

from . import cmpattn as _cmp
from . import selattn as _sel

LOG2E = 1.4426950408889634


def _bounds(cu):
    cu = [int(x) for x in cu]
    return [(cu[i], cu[i + 1]) for i in range(len(cu) - 1)]


def window_attention_ref(q, k, v, cu_seqlens, window: int, softmax_scale=None, dtype=torch.float32):
    """(O [N,Hq,D], base-2 LSE [Hq,N]); differentiable."""
    N, Hq, D = q.shape
    Hkv = k.shape[1]
    g = Hq // Hkv
    if softmax_scale is None:
        softmax_scale = 1.0 / math.sqrt(D)
    outs, lses = [], []
    for (s0, s1) in _bounds(cu_seqlens):
        L = s1 - s0
        i = torch.arange(L)[:, None]
        p = torch.arange(L)[None, :]
        vis = (p <= i) & (p >= i - window)
        kx = k[s0:s1].to(dtype).repeat_interleave(g, dim=1)
        vx = v[s0:s1].to(dtype).repeat_interleave(g, dim=1)
        s = torch.einsum("ihd,phd->hip", q[s0:s1].to(dtype), kx) * softmax_scale
        s = s.masked_fill(~vis[None], float("-inf"))
        outs.append(torch.einsum("hip,phd->ihd", torch.softmax(s, -1), vx))
        lses.append(torch.logsumexp(s, -1) * LOG2E)
    return torch.cat(outs, 0), torch.cat(lses, 1)


def llama3_inv_freq(head_dim: int, theta: float, factor: float = 8.0, low_freq_factor: float = 1.0,
                    high_freq_factor: float = 4.0, original_max: int = 8192) -> torch.Tensor:
    """fp32 [D/2] frequency table of the "llama3" rope scaling."""
    inv = 1.0 / (theta ** (torch.arange(0, head_dim, 2, dtype=torch.int64).float() / head_dim))
    low_wl = original_max / low_freq_factor
    high_wl = original_max / high_freq_factor
    wl = 2 * math.pi / inv
    out = torch.where(wl > low_wl, inv / factor, inv)
    smooth = (original_max / wl - low_freq_factor) / (high_freq_factor - low_freq_factor)
    mid = (1 - smooth) * out / factor + smooth * out
    is_mid = ~(wl < high_wl) & ~(wl > low_wl)
    return torch.where(is_mid, mid, out)


def rope_ref(x, cu_seqlens, inv_freq, start: int = 0, stride: int = 1, table_dtype=None, conj: bool = False):
    """Rotary embedding on packed sequences: token j of a sequence sits at position
    start + j*stride (nsa_ref/module/rope.py:126-134).  cos/sin are computed in fp32 and
    rounded to `table_dtype` (the reference rounds them to x.dtype, rope.py:124) before a
    fp32 rotation.  conj=True applies the inverse rotation (= the backward of the forward)."""
    N, H, D = x.shape
    out = torch.empty_like(x, dtype=torch.float32)
    for (s0, s1) in _bounds(cu_seqlens):
        pos = (start + torch.arange(s1 - s0) * stride).float()
        ang = pos[:, None] * inv_freq.float()[None, :]
        cos, sin = ang.cos(), ang.sin()
        if table_dtype is not None:
            cos, sin = cos.to(table_dtype).float(), sin.to(table_dtype).float()
        if conj:
            sin = -sin
        x1, x2 = x[s0:s1, :, : D // 2].float(), x[s0:s1, :, D // 2:].float()
        out[s0:s1, :, : D // 2] = x1 * cos[:, None] - x2 * sin[:, None]
        out[s0:s1, :, D // 2:] = x1 * sin[:, None] + x2 * cos[:, None]
    return out


def fsa_layer_ref(params: dict, x, cu_seqlens, cfg: dict, topk_idx=None, table_dtype=None):
    """fp32 composition of the layer (fsa/module/fsa.py:71-173).  `params` holds the reference's
    parameter names; `cfg` the constructor arguments plus "inv_freq".  When `topk_idx` is given it
    replaces the selection computed from the compressed branch (the selection is discrete, so a
    like-for-like comparison passes the ids the device chose).  Returns (y, topk_idx, parts);
    parts["block_score"] holds the fp32 block scores [Hkv, N, nblk] when the selection was computed here."""
    hq, hkv, d = cfg["num_q_heads"], cfg["num_kv_heads"], cfg["head_dim"]
    ks, st, bk, t = cfg["kernel_size"], cfg["kernel_stride"], cfg["block_size"], cfg["topk"]
    xf = x.float()
    q = (xf @ params["proj_q.weight"].float().t()).view(-1, hq, d)
    k = (xf @ params["proj_k.weight"].float().t()).view(-1, hkv, d)
    v = (xf @ params["proj_v.weight"].float().t()).view(-1, hkv, d)
    ck, cu_k = _cmp.linear_compress_ref(k, params["compress_key"].float(), cu_seqlens, ks, st,
                                        params["intra_block_pe"].float())
    cv, _ = _cmp.linear_compress_ref(v, params["compress_value"].float(), cu_seqlens, ks, st, None)
    inv = cfg["inv_freq"]

    def rope(z, cu, start=0, stride=1):
        # differentiable rotation (rope_ref writes in place, so restate it functionally here)
        outs = []
        for (s0, s1) in _bounds(cu):
            pos = (start + torch.arange(s1 - s0) * stride).float()
            ang = pos[:, None] * inv.float()[None, :]
            cos, sin = ang.cos(), ang.sin()
            if table_dtype is not None:
                cos, sin = cos.to(table_dtype).float(), sin.to(table_dtype).float()
            z1, z2 = z[s0:s1, :, : d // 2], z[s0:s1, :, d // 2:]
            outs.append(torch.cat([z1 * cos[:, None] - z2 * sin[:, None], z1 * sin[:, None] + z2 * cos[:, None]], -1))
        return torch.cat(outs, 0) if outs else z

    q = rope(q, cu_seqlens)
    ck = rope(ck, cu_k, 0, st)
    o_cmp, lse_cmp = _cmp.compressed_attention_ref(q, ck, cv, ks, st, cu_seqlens, cu_k)
    block_score = None
    if topk_idx is None:
        max_q = max(b - a for a, b in _bounds(cu_seqlens))
        topk_idx, block_score = _cmp.compressed_topk_ref(q.detach(), ck.detach(), lse_cmp.detach(), ks, st, bk, t,
                                                         cu_seqlens, cu_k, init_blocks=cfg["init_blocks"],
                                                         local_blocks=cfg["local_blocks"], max_seqlen_q=max_q)
    k = rope(k, cu_seqlens)
    o_sel, _ = _sel.selected_attention_ref(q, k, v, topk_idx, bk, cu_seqlens)
    o_win, _ = window_attention_ref(q, k, v, cu_seqlens, cfg["window_size"])
    gate = torch.sigmoid(xf @ params["gate.0.weight"].float().t())
    o = gate[:, 0:1, None] * o_cmp + gate[:, 1:2, None] * o_sel + gate[:, 2:3, None] * o_win
    y = o.reshape(o.shape[0], -1) @ params["proj_o.weight"].float().t()
    return y, topk_idx, {"cmp": o_cmp, "sel": o_sel, "win": o_win, "gate": gate, "block_score": block_score}
