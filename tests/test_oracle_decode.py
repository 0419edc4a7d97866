"""Pins the decode oracle: on a consistent cache the decode step for the last
token must reproduce the last row of the (already pinned) prefill oracles."""
import math

import torch

from synth_inputs import make_topk_idx
from oracle import cmpattn as pre
from oracle import decode as dec
from oracle import selattn as sel

KS, ST, BK, T = 8, 4, 16, 4


def _setup(lens=(300, 77, 130), hq=4, hkv=2, d=16, seed=0):
    gen = torch.Generator().manual_seed(seed)
    cu = [0]
    for l in lens:
        cu.append(cu[-1] + l)
    n = cu[-1]
    q = torch.randn(n, hq, d, generator=gen, dtype=torch.float64)
    k = torch.randn(n, hkv, d, generator=gen, dtype=torch.float64)
    v = torch.randn(n, hkv, d, generator=gen, dtype=torch.float64)
    wk = torch.randn(hkv, KS * d, d, generator=gen, dtype=torch.float64) / math.sqrt(KS * d)
    ck, cu_ck = pre.linear_compress_ref(k, wk, cu, KS, ST, dtype=torch.float64)
    cv, _ = pre.linear_compress_ref(v, wk.flip(0), cu, KS, ST, dtype=torch.float64)
    last = torch.tensor([c - 1 for c in cu[1:]])
    return cu, q, k, v, ck, cv, cu_ck, last


def test_decode_compressed_attention_is_last_prefill_row():
    cu, q, k, v, ck, cv, cu_ck, last = _setup()
    o_p, lse_p = pre.compressed_attention_ref(q, ck, cv, KS, ST, cu, cu_ck, dtype=torch.float64)
    pos = torch.tensor([cu[i + 1] - cu[i] - 1 for i in range(len(cu) - 1)])
    o_d, lse_d = dec.decode_compressed_attention_ref(q[last], ck, cv, cu_ck, pos, KS, ST, dtype=torch.float64)
    assert torch.allclose(o_d, o_p[last], atol=1e-12)
    assert torch.allclose(lse_d, lse_p[:, last], atol=1e-12)


def test_decode_block_scores_and_topk_are_last_prefill_row():
    cu, q, k, v, ck, cv, cu_ck, last = _setup()
    _, lse_p = pre.compressed_attention_ref(q, ck, cv, KS, ST, cu, cu_ck, dtype=torch.float64)
    lens = [cu[i + 1] - cu[i] for i in range(len(cu) - 1)]
    pos = torch.tensor([l - 1 for l in lens])
    for b in range(len(lens)):  # one request at a time: the prefill matrix width follows its longest sequence
        cu1, cuk1 = [0, lens[b]], [0, cu_ck[b + 1] - cu_ck[b]]
        sl, slk = slice(cu[b], cu[b + 1]), slice(cu_ck[b], cu_ck[b + 1])
        idx_p, bs_p = pre.compressed_topk_ref(q[sl], ck[slk], lse_p[:, sl].float(), KS, ST, BK, T, cu1, cuk1,
                                              to_bf16=False)
        bs_d = dec.decode_block_scores_ref(q[last[b:b + 1]], ck[slk], lse_p[:, last[b:b + 1]].float(), cuk1,
                                           pos[b:b + 1], [lens[b]], KS, ST, BK)
        assert torch.allclose(bs_d[:, 0], bs_p[:, -1], atol=1e-6)
        got = dec.decode_topk_ref(bs_d, T)[:, 0].sort(-1).values
        want = idx_p[:, -1].sort(-1).values
        assert torch.equal(got, want)


def test_decode_block_scores_as_written_brute_force():
    cu, q, k, v, ck, cv, cu_ck, last = _setup(lens=(300,))
    pos = torch.tensor([299])
    _, lse = dec.decode_compressed_attention_ref(q[last], ck, cv, cu_ck, pos, KS, ST, dtype=torch.float64)
    bs = dec.decode_block_scores_ref(q[last], ck, lse.float(), cu_ck, pos, [300], KS, ST, BK, as_written=True)
    nc = cu_ck[1]
    assert bs.shape[-1] == math.ceil(nc / BK)          # candidate blocks counted from the COMPRESSED length
    assert torch.isinf(bs[:, 0, 0]).all() and (bs[:, 0, 0] > 0).all()   # block 0: init block and "own" block
    assert torch.isfinite(bs[:, 0, 1:]).all()          # nothing else is forced
    # kv head 1 scores q-head 1 (not q-head 2 = first head of its group)
    s = (ck[:nc, 1].float() @ q[last[0], 1].float()) * (pre.LOG2E / 4.0)
    p = torch.exp2(s - lse[1, 0].float())
    blk = 2
    want = p[7] + 2 * p[8] + 2 * p[9] + 2 * p[10] + p[11]
    assert abs(float(bs[1, 0, blk]) - float(want)) < 1e-6


def test_decode_selected_attention_is_last_prefill_row():
    cu, q, k, v, ck, cv, cu_ck, last = _setup()
    topk = make_topk_idx(cu, 2, BK, T, seed=3)
    o_p, lse_p = sel.selected_attention_ref(q, k, v, topk, BK, cu, dtype=torch.float64)
    o_d, lse_d = dec.decode_selected_attention_ref(q[last], k, v, cu, topk[:, last], BK, dtype=torch.float64)
    assert torch.allclose(o_d, o_p[last], atol=1e-12)
    assert torch.allclose(lse_d, lse_p[:, last], atol=1e-12)
    # -1 padding, ids past the cache and duplicates are ignored
    noisy = torch.cat([topk[:, last], torch.full_like(topk[:, last], -1), topk[:, last][..., :1]], -1)
    noisy[0, 0, T] = 10 ** 6
    o_n, _ = dec.decode_selected_attention_ref(q[last], k, v, cu, noisy, BK, dtype=torch.float64)
    assert torch.allclose(o_n, o_d, atol=1e-12)


def test_as_written_selected_closed_form():
    cu, q, k, v, ck, cv, cu_ck, last = _setup()
    o, lse = dec.as_written_selected_ref(q[last], k, v, cu, dtype=torch.float64)
    only0 = torch.zeros(2, 3, 1, dtype=torch.int32)
    # attending to block 0 of a cache truncated to one token is the same thing
    cu1 = [0, 1, 2, 3]
    first = torch.tensor(cu[:-1])
    o2, lse2 = dec.decode_selected_attention_ref(q[last], k[first], v[first], cu1, only0, BK, dtype=torch.float64)
    assert torch.allclose(o, o2, atol=1e-12) and torch.allclose(lse, lse2, atol=1e-12)
