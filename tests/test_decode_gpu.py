"""GPU parity: one-step decode kernels vs the CPU oracle (batch of requests).

Tolerances: O max-abs 2e-2 (bf16) / 5e-3 (fp16), base-2 LSE 1e-3; selected block
ids bit-exact given the block scores the kernel produced.
"""
import math

import pytest
import torch

from fsa_hip import ops
from oracle import decode as orc

pytestmark = pytest.mark.gpu
TOL = {torch.bfloat16: 2e-2, torch.float16: 5e-3}
KS, ST = 32, 16


def _caches(lens, hq, hkv, d, dtype, seed, raw=True):
    gen = torch.Generator().manual_seed(seed)
    b = len(lens)
    cu_k = [0]
    cu_ck = [0]
    for l in lens:
        cu_k.append(cu_k[-1] + l)
        cu_ck.append(cu_ck[-1] + ((l - KS) // ST + 1 if l >= KS else 0))
    std = 0.5 if d == 256 else 1.0
    q = (torch.randn(b, hq, d, generator=gen) * std).to(dtype)
    kc = (torch.randn(cu_k[-1], hkv, d, generator=gen) * std).to(dtype) if raw else None
    vc = (torch.randn(cu_k[-1], hkv, d, generator=gen) * std).to(dtype) if raw else None
    ck = (torch.randn(max(cu_ck[-1], 1), hkv, d, generator=gen) * std).to(dtype)
    cv = (torch.randn(max(cu_ck[-1], 1), hkv, d, generator=gen) * std).to(dtype)
    return q, kc, vc, ck, cv, cu_k, cu_ck


CASES = [
    # cache lengths (new token included), Hq, Hkv, D, B_K, T, dtype
    ([4000, 70, 33, 1025, 2600], 8, 2, 128, 64, 16, torch.bfloat16),
    ([31, 5000], 4, 4, 128, 64, 16, torch.bfloat16),              # first request has no compressed key
    ([3000, 900, 1500], 6, 2, 64, 32, 8, torch.float16),          # g = 3, block 32
    ([2048, 4100], 4, 2, 256, 128, 8, torch.float16),
    ([1300, 40, 2600], 32, 2, 128, 64, 8, torch.bfloat16),        # GQA group of 16: one launch, or 15 + 1 heads
    ([900, 3000], 20, 1, 64, 64, 8, torch.float16),               # GQA group of 20: two launches
]


def _many_lens(n, lo, hi, seed):
    gen = torch.Generator().manual_seed(seed)
    return torch.randint(lo, hi + 1, (n,), generator=gen).tolist()


# Many requests: the tile sequence is longer than the persistent grid, so a wave's share holds several tiles and
# crosses (request, kv head) boundaries, requests without any compressed key included.
MANY_COMPRESSED = (_many_lens(120, 16, 40000, 77), 8, 2, 128, 64, 16, torch.bfloat16)
MANY_SELECTED = (_many_lens(300, 40, 1500, 78), 8, 2, 128, 64, 16, torch.bfloat16)


@pytest.mark.parametrize("lens,hq,hkv,d,bk,t,dtype", CASES + [MANY_COMPRESSED])
@pytest.mark.parametrize("as_written", [False, True])
def test_decode_compressed_and_topk(dev, lens, hq, hkv, d, bk, t, dtype, as_written):
    print(f"case lens={lens[:8]}{'...' if len(lens) > 8 else ''} ({len(lens)} requests) hq={hq} hkv={hkv} d={d} bk={bk} "
          f"t={t} {dtype} as_written={as_written}", flush=True)
    q, kc, vc, ck, cv, cu_k, cu_ck = _caches(lens, hq, hkv, d, dtype, seed=21, raw=False)
    pos = torch.tensor([l - 1 for l in lens], dtype=torch.int32)
    seqlens = torch.tensor(lens, dtype=torch.int32)
    max_ck = max(b_ - a_ for a_, b_ in zip(cu_ck[:-1], cu_ck[1:]))
    cu_ck_t = torch.tensor(cu_ck, dtype=torch.int32, device=dev)
    o, lse, raw = ops.decode_cmpattn(q.to(dev), ck.to(dev), cv.to(dev), cu_ck_t, pos.to(dev), KS, ST, max_ck,
                                     score_head_as_written=as_written)
    nblk_max = max(math.ceil((c1 - c0) / bk) if as_written else math.ceil(l / bk)
                   for l, c0, c1 in zip(lens, cu_ck[:-1], cu_ck[1:]))
    nblk_max = max(nblk_max, 1)
    idx, bscore = ops.decode_topk(raw, lse, cu_ck_t, pos.to(dev), seqlens.to(dev), hq, KS, ST, bk, t, nblk_max,
                                  softmax_scale=1.0 / math.sqrt(d), as_written=as_written,
                                  return_block_score=True)
    torch.cuda.synchronize()
    o_r, lse_r = orc.decode_compressed_attention_ref(q.float(), ck.float(), cv.float(), cu_ck, pos, KS, ST)
    lse_c = lse.cpu()
    dead = torch.isinf(lse_r)
    assert torch.equal(torch.isinf(lse_c) & (lse_c < 0), dead)
    if (~dead).any():
        assert (lse_c[~dead] - lse_r[~dead]).abs().max().item() <= 1e-3
    err = (o.float().cpu() - o_r).abs().max().item()
    print(f"  max|dO|={err:.3e}", flush=True)
    assert err <= TOL[dtype]
    # selection bit-exact given the kernel's block scores
    bscore, idx = bscore.cpu(), idx.cpu()
    assert torch.equal(idx, orc.decode_topk_ref(bscore, t))
    # ... and with the scores rounded to bf16 before ranking (the prefill layer's rule; -inf slots stay -inf)
    idx16 = ops.decode_topk(raw, lse, cu_ck_t, pos.to(dev), seqlens.to(dev), hq, KS, ST, bk, t, nblk_max,
                            softmax_scale=1.0 / math.sqrt(d), as_written=as_written, scores_to_bf16=True)
    assert torch.equal(idx16.cpu(), orc.decode_topk_ref(bscore.to(torch.bfloat16).float(), t))
    # block scores vs the oracle
    bs_r = orc.decode_block_scores_ref(q.float(), ck.float(), lse_r, cu_ck, pos, lens, KS, ST, bk,
                                       as_written=as_written, nblk_cols=nblk_max)
    assert torch.equal(torch.isinf(bscore), torch.isinf(bs_r))
    fin = torch.isfinite(bs_r)
    diff = (bscore[fin] - bs_r[fin]).abs().max().item() if fin.any() else 0.0
    print(f"  block-score max diff {diff:.3e}", flush=True)
    assert diff <= 2e-3


@pytest.mark.parametrize("lens,hq,hkv,d,bk,t,dtype", CASES + [MANY_SELECTED])
def test_decode_selected(dev, lens, hq, hkv, d, bk, t, dtype):
    print(f"case lens={lens[:8]}{'...' if len(lens) > 8 else ''} ({len(lens)} requests) hq={hq} hkv={hkv} d={d} bk={bk} "
          f"t={t} {dtype}", flush=True)
    q, kc, vc, ck, cv, cu_k, cu_ck = _caches(lens, hq, hkv, d, dtype, seed=22)
    gen = torch.Generator().manual_seed(5)
    b = len(lens)
    topk = torch.full((hkv, b, t), -1, dtype=torch.int32)
    for i, l in enumerate(lens):
        nb = math.ceil(l / bk)
        for h in range(hkv):
            pick = torch.randperm(nb, generator=gen)[: min(t, nb)]
            topk[h, i, : pick.numel()] = pick.to(torch.int32)
    topk[0, 0, -1] = topk[0, 0, 0]          # a repeated id
    if t > 2:
        topk[-1, -1, 1] = 10 ** 6           # an id past the cache
    cu_k_t = torch.tensor(cu_k, dtype=torch.int32, device=dev)
    o, lse = ops.decode_selattn(q.to(dev), kc.to(dev), vc.to(dev), cu_k_t, topk.to(dev), bk)
    torch.cuda.synchronize()
    o_r, lse_r = orc.decode_selected_attention_ref(q.float(), kc.float(), vc.float(), cu_k, topk, bk)
    err = (o.float().cpu() - o_r).abs().max().item()
    err_l = (lse.cpu() - lse_r).abs().max().item()
    print(f"  max|dO|={err:.3e} max|dLSE|={err_l:.3e}", flush=True)
    assert err <= TOL[dtype] and err_l <= 1e-3
    # the reference's call as written keeps key 0 only: block 0 of a one-token cache
    first = torch.tensor(cu_k[:-1])
    cu1 = torch.arange(b + 1, dtype=torch.int32, device=dev)
    only0 = torch.zeros((hkv, b, 1), dtype=torch.int32, device=dev)
    o_w, lse_w = ops.decode_selattn(q.to(dev), kc[first].to(dev), vc[first].to(dev), cu1, only0, bk)
    o_wr, lse_wr = orc.as_written_selected_ref(q.float(), kc.float(), vc.float(), cu_k)
    assert (o_w.float().cpu() - o_wr).abs().max().item() <= 1e-6
    assert (lse_w.cpu() - lse_wr).abs().max().item() <= 1e-3


@pytest.mark.parametrize("ks,st,bk", [(64, 16, 64), (16, 16, 32), (32, 8, 64)])
def test_decode_other_geometries(dev, monkeypatch, ks, st, bk):
    """Compression windows / strides / block sizes other than 32 / 16 / 64 (other tap weights of the re-binning)."""
    import sys
    me = sys.modules[__name__]
    monkeypatch.setattr(me, "KS", ks)
    monkeypatch.setattr(me, "ST", st)
    lens = [3000, 100, ks - 1, 1700]
    test_decode_compressed_and_topk(dev, lens, 8, 2, 128, bk, 8, torch.bfloat16, False)
    test_decode_selected(dev, lens, 8, 2, 128, bk, 8, torch.bfloat16)
