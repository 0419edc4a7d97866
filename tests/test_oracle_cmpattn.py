"""Pins the compressed-attention / block-score / top-k oracle without the reference."""
import math

import pytest
import torch
import torch.nn.functional as F

from oracle import cmpattn as orc

KS, ST, BK = 8, 4, 16  # kernel_size, kernel_stride, block_size (same ratios as 32/16/64)


def _inputs(cu, hq=4, hkv=2, d=16, seed=0, dtype=torch.float64):
    gen = torch.Generator().manual_seed(seed)
    n = cu[-1]
    q = torch.randn(n, hq, d, generator=gen, dtype=dtype)
    k = torch.randn(n, hkv, d, generator=gen, dtype=dtype)
    v = torch.randn(n, hkv, d, generator=gen, dtype=dtype)
    wk = torch.randn(hkv, KS * d, d, generator=gen, dtype=dtype) / math.sqrt(KS * d)
    wv = torch.randn(hkv, KS * d, d, generator=gen, dtype=dtype) / math.sqrt(KS * d)
    pe = torch.randn(hkv, KS, d, generator=gen, dtype=dtype)
    return q, k, v, wk, wv, pe


def test_compressed_lens_and_linear_compress_brute_force():
    cu = [0, 5, 45, 53, 120]  # first sequence shorter than the kernel, third exactly one window
    q, k, v, wk, wv, pe = _inputs(cu)
    assert orc.compressed_lens(cu, KS, ST) == [0, 0, 9, 10, 25]
    y, cu_y = orc.linear_compress_ref(k, wk, cu, KS, ST, pe, dtype=torch.float64)
    assert y.shape[0] == cu_y[-1]
    W = wk.reshape(2, KS, 16, 16)
    for s in range(4):
        for j in range(cu_y[s + 1] - cu_y[s]):
            for h in range(2):
                acc = torch.zeros(16, dtype=torch.float64)
                for kk in range(KS):
                    acc += (k[cu[s] + j * ST + kk, h] + pe[h, kk]) @ W[h, kk]
                assert torch.allclose(y[cu_y[s] + j, h], acc, atol=1e-12)


@pytest.mark.parametrize("cu", [[0, 96], [0, 5, 45, 53, 120]])
def test_compressed_attention_matches_sdpa_and_closed_forms(cu):
    q, k, v, wk, wv, pe = _inputs(cu)
    ck, cu_k = orc.linear_compress_ref(k, wk, cu, KS, ST, pe, dtype=torch.float64)
    cv, _ = orc.linear_compress_ref(v, wv, cu, KS, ST, None, dtype=torch.float64)
    o, lse = orc.compressed_attention_ref(q, ck, cv, KS, ST, cu, cu_k, dtype=torch.float64)
    for s in range(len(cu) - 1):
        q0, q1, k0, k1 = cu[s], cu[s + 1], cu_k[s], cu_k[s + 1]
        L, nc = q1 - q0, k1 - k0
        # queries before kernel_size - 1 (or with no compressed key at all): O = 0, LSE = -inf
        dead = min(L, KS - 1) if nc > 0 else L
        assert (o[q0:q0 + dead] == 0).all() and torch.isinf(lse[:, q0:q0 + dead]).all()
        if nc == 0:
            continue
        vis = orc.visible_mask(L, nc, KS, ST)
        live = vis.any(-1)
        kx, vx = ck[k0:k1].repeat_interleave(2, 1), cv[k0:k1].repeat_interleave(2, 1)
        ref = F.scaled_dot_product_attention(q[q0:q1].transpose(0, 1)[None], kx.transpose(0, 1)[None],
                                             vx.transpose(0, 1)[None], attn_mask=vis[None, None])[0].transpose(0, 1)
        assert torch.allclose(o[q0:q1][live], ref[live], atol=1e-10)
        # first live query (position ks - 1) sees exactly compressed key 0
        i = KS - 1
        for h in range(4):
            assert torch.allclose(o[q0 + i, h], cv[k0, h // 2], atol=1e-12)
            want = orc.LOG2E * float(q[q0 + i, h] @ ck[k0, h // 2]) / math.sqrt(16)
            assert abs(lse[h, q0 + i].item() - want) < 1e-10


def test_score_is_softmax_probability_of_first_group_head():
    cu = [0, 5, 45, 53, 120]
    q, k, v, wk, wv, pe = _inputs(cu)
    ck, cu_k = orc.linear_compress_ref(k, wk, cu, KS, ST, pe, dtype=torch.float64)
    cv, _ = orc.linear_compress_ref(v, wv, cu, KS, ST, None, dtype=torch.float64)
    _, lse = orc.compressed_attention_ref(q, ck, cv, KS, ST, cu, cu_k, dtype=torch.float64)
    sc = orc.attention_score_ref(q, ck, lse, KS, ST, cu, cu_k, dtype=torch.float64)
    assert sc.shape == (2, 120, 15)  # max per-sequence compressed length
    for s in range(4):
        q0, q1, nc = cu[s], cu[s + 1], cu_k[s + 1] - cu_k[s]
        rows = sc[:, q0:q1].sum(-1)
        live = torch.arange(q1 - q0) >= KS - 1 if nc > 0 else torch.zeros(q1 - q0, dtype=torch.bool)
        assert torch.allclose(rows[:, live], torch.ones_like(rows[:, live]), atol=1e-10)
        assert (rows[:, ~live] == 0).all()
        assert (sc[:, q0:q1, nc:] == 0).all()
        if nc:
            # head kh*g, not the group mean: compare with an explicit softmax of that head
            vis = orc.visible_mask(q1 - q0, nc, KS, ST)
            for kh in range(2):
                s_ = (q[q0:q1, kh * 2] @ ck[cu_k[s]:cu_k[s + 1], kh].t()) / 4.0
                p = torch.softmax(s_.masked_fill(~vis, float("-inf")), -1)
                assert torch.allclose(sc[kh, q0:q1, :nc][live], p[live], atol=1e-10)


def test_transform_weights_and_brute_force():
    assert orc.score_weights(32, 16, 64).tolist() == [1, 2, 2, 2, 1]
    assert orc.score_weights(KS, ST, BK).tolist() == [1, 2, 2, 2, 1]
    cu = [0, 45, 120]
    gen = torch.Generator().manual_seed(1)
    score = torch.rand(2, 120, 17, generator=gen, dtype=torch.float64)
    out = orc.transform_score_ref(score, KS, ST, BK, cu, init_blocks=1, local_blocks=2)
    nblk = math.ceil(75 / BK)
    assert out.shape == (2, 120, nblk)
    w = [1, 2, 2, 2, 1]
    for (q0, q1) in ((0, 45), (45, 120)):
        for i in (0, 7, 16, 31, 44, q1 - q0 - 1):
            bq = i // BK
            for b in range(nblk):
                if b < 1 or (bq - 2 < b <= bq):
                    assert torch.isinf(out[:, q0 + i, b]).all()
                    continue
                acc = torch.zeros(2, dtype=torch.float64)
                for o_ in range(5):
                    col = b * (BK // ST) - (KS // ST - 1) + o_
                    if 0 <= col < 17:
                        acc += w[o_] * score[:, q0 + i, col]
                assert torch.allclose(out[:, q0 + i, b], acc, atol=1e-12)


def test_topk_select_matches_torch_topk_without_ties():
    cu = [0, 300, 700]
    gen = torch.Generator().manual_seed(2)
    nblk = math.ceil(400 / BK)
    bs = torch.rand(2, 700, nblk, generator=gen)
    bs[:, :, 0] = float("inf")
    got = orc.topk_select_ref(bs, 6, cu, BK, to_bf16=True)
    ties = orc.kth_value_tie_rows(bs, 6, to_bf16=True)
    sc = bs.to(torch.bfloat16)
    ref = sc.topk(6, dim=-1, sorted=False).indices.sort(-1).values
    q_idx = torch.cat([torch.arange(300) // BK, torch.arange(400) // BK])
    ref[ref > q_idx[None, :, None]] = -1
    ref = ref.to(torch.int32)
    assert ties.float().mean() < 0.5
    assert torch.equal(got[~ties], ref[~ties])
    # rows with a tie at the k-th value: same multiset of selected VALUES, ids by lower index first
    assert got.dtype == torch.int32 and got.shape == (2, 700, 6)
    # ascending with -1 only above the own block, and -1s trailing after the sort+mask
    valid = got >= 0
    assert (got[valid] <= q_idx[None, :, None].expand_as(got)[valid]).all()


def test_compressed_grads_match_dense_autograd():
    cu = [0, 45, 53, 120]
    q, k, v, wk, wv, pe = _inputs(cu)
    ck, cu_k = orc.linear_compress_ref(k, wk, cu, KS, ST, pe, dtype=torch.float64)
    cv, _ = orc.linear_compress_ref(v, wv, cu, KS, ST, None, dtype=torch.float64)
    do = torch.randn(120, 4, 16, dtype=torch.float64, generator=torch.Generator().manual_seed(9))
    o, lse, dq, dk, dv = orc.compressed_attention_grads_ref(q, ck, cv, KS, ST, cu, cu_k, do, dtype=torch.float64)
    # explicit formulas on one sequence / head
    q0, q1, k0, k1 = 53, 120, cu_k[2], cu_k[3]
    vis = orc.visible_mask(q1 - q0, k1 - k0, KS, ST)
    h, kh = 3, 1
    s = (q[q0:q1, h] @ ck[k0:k1, kh].t()) / 4.0
    p = torch.softmax(s.masked_fill(~vis, float("-inf")), -1)
    p = torch.where(vis.any(-1, keepdim=True), p, torch.zeros_like(p))
    dp = do[q0:q1, h] @ cv[k0:k1, kh].t()
    delta = (o[q0:q1, h] * do[q0:q1, h]).sum(-1, keepdim=True)
    ds = p * (dp - delta) / 4.0
    assert torch.allclose(dq[q0:q1, h], ds @ ck[k0:k1, kh], atol=1e-10)
    # the explicit-formula path (used with bf16 / fp16 rounding points) equals autograd when the
    # rounding is the identity
    o2, lse2, dq2, dk2, dv2 = orc.compressed_attention_grads_ref(q, ck, cv, KS, ST, cu, cu_k, do,
                                                                 dtype=torch.float64, round_dtype=torch.float64)
    assert torch.allclose(dq2, dq, atol=1e-10) and torch.allclose(dk2, dk, atol=1e-10)
    assert torch.allclose(dv2, dv, atol=1e-10)
