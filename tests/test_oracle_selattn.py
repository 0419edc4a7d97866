"""Pins the selected-attention oracle without the reference: dense-mask fp64
softmax, a library routine (SDPA with a bool mask), closed forms, invariants,
finite differences and brute-force index construction."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from synth_inputs import make_qkv, make_topk_idx
from oracle import selattn as orc


def _case(n=300, hq=4, hkv=2, d=32, bk=16, t=4, seed=0, cu=None):
    cu = cu or [0, n]
    q, k, v, do = make_qkv(cu[-1], hq, hkv, d, torch.float64, seed=seed)
    topk = make_topk_idx(cu, hkv, bk, t, seed=seed + 1)
    return cu, q, k, v, do, topk


@pytest.mark.parametrize("cu", [[0, 300], [0, 100, 101, 260, 300]])
def test_gather_oracle_equals_dense_softmax(cu):
    cu, q, k, v, do, topk = _case(cu=cu)
    o, lse = orc.selected_attention_ref(q, k, v, topk, 16, cu, dtype=torch.float64, q_chunk=37)
    o_d, lse_d = orc.selected_attention_dense_ref(q, k, v, topk, 16, cu)
    assert torch.allclose(o, o_d, atol=1e-12)
    assert torch.allclose(lse, lse_d, atol=1e-12)


def test_oracle_equals_sdpa_with_bool_mask():
    cu, q, k, v, do, topk = _case(n=256, hq=4, hkv=2, d=32)
    o, _ = orc.selected_attention_ref(q, k, v, topk, 16, cu, dtype=torch.float64)
    mask = orc.dense_mask(topk, 16, cu).repeat_interleave(2, dim=0)  # [Hq, N, N]
    kx, vx = k.repeat_interleave(2, dim=1), v.repeat_interleave(2, dim=1)
    o_sdpa = F.scaled_dot_product_attention(q.transpose(0, 1)[None], kx.transpose(0, 1)[None],
                                            vx.transpose(0, 1)[None], attn_mask=mask[None])
    assert torch.allclose(o, o_sdpa[0].transpose(0, 1), atol=1e-10)


def test_all_blocks_selected_is_plain_causal_attention():
    n, bk = 128, 16
    cu, q, k, v, do, _ = _case(n=n, bk=bk)
    nb = n // bk
    topk = torch.arange(nb, dtype=torch.int32)[None, None, :].expand(2, n, nb).contiguous()
    o, lse = orc.selected_attention_ref(q, k, v, topk, bk, cu, dtype=torch.float64)
    kx, vx = k.repeat_interleave(2, dim=1), v.repeat_interleave(2, dim=1)
    o_c = F.scaled_dot_product_attention(q.transpose(0, 1)[None], kx.transpose(0, 1)[None],
                                         vx.transpose(0, 1)[None], is_causal=True)[0].transpose(0, 1)
    assert torch.allclose(o, o_c, atol=1e-10)
    s = torch.einsum("ihd,phd->hip", q, kx) / math.sqrt(q.shape[-1])
    s = s.masked_fill(torch.ones(n, n).tril() == 0, float("-inf"))
    assert torch.allclose(lse, torch.logsumexp(s, -1) * orc.LOG2E, atol=1e-10)


def test_own_block_only_is_block_diagonal_causal():
    n, bk = 96, 16
    cu, q, k, v, do, _ = _case(n=n, bk=bk)
    own = (torch.arange(n) // bk).to(torch.int32)
    topk = torch.full((2, n, 3), -1, dtype=torch.int32)
    topk[:, :, 0] = own
    o, _ = orc.selected_attention_ref(q, k, v, topk, bk, cu, dtype=torch.float64)
    for b in range(n // bk):
        sl = slice(b * bk, (b + 1) * bk)
        kx, vx = k[sl].repeat_interleave(2, dim=1), v[sl].repeat_interleave(2, dim=1)
        o_b = F.scaled_dot_product_attention(q[sl].transpose(0, 1)[None], kx.transpose(0, 1)[None],
                                             vx.transpose(0, 1)[None], is_causal=True)[0].transpose(0, 1)
        assert torch.allclose(o[sl], o_b, atol=1e-10)


def test_token_zero_closed_form_and_scale():
    cu, q, k, v, do, topk = _case()
    scale = 0.37
    o, lse = orc.selected_attention_ref(q, k, v, topk, 16, cu, softmax_scale=scale, dtype=torch.float64)
    # token 0 sees key 0 only: O = v[0, kh], LSE2 = log2(e) * scale * q0.k0
    for h in range(4):
        assert torch.allclose(o[0, h], v[0, h // 2], atol=1e-12)
        assert abs(lse[h, 0].item() - orc.LOG2E * scale * float(q[0, h] @ k[0, h // 2])) < 1e-12


def test_slot_permutation_and_padding_invariance():
    cu, q, k, v, do, topk = _case()
    o, lse = orc.selected_attention_ref(q, k, v, topk, 16, cu, dtype=torch.float64)
    perm = torch.tensor([2, 0, 3, 1])
    wide = torch.cat([topk[:, :, perm], torch.full_like(topk, -1)], dim=-1)
    o2, lse2 = orc.selected_attention_ref(q, k, v, wide, 16, cu, dtype=torch.float64)
    assert torch.allclose(o, o2, atol=1e-12) and torch.allclose(lse, lse2, atol=1e-12)


def test_grads_match_dense_autograd_and_finite_differences():
    cu, q, k, v, do, topk = _case(n=48, hq=4, hkv=2, d=8, bk=8, t=3, cu=[0, 30, 48])
    o, lse, dq, dk, dv = orc.selected_attention_grads_ref(q, k, v, topk, 8, cu, do, dtype=torch.float64)
    qd, kd, vd = (x.clone().requires_grad_(True) for x in (q, k, v))
    od, _ = orc.selected_attention_dense_ref(qd, kd, vd, topk, 8, cu)
    (od * do).sum().backward()
    assert torch.allclose(dq, qd.grad, atol=1e-11)
    assert torch.allclose(dk, kd.grad, atol=1e-11)
    assert torch.allclose(dv, vd.grad, atol=1e-11)
    assert torch.allclose(o, od, atol=1e-12)
    # and against autograd through the gather formulation
    qg, kg, vg = (x.clone().requires_grad_(True) for x in (q, k, v))
    og, lseg = orc.selected_attention_ref(qg, kg, vg, topk, 8, cu, dtype=torch.float64)
    (og * do).sum().backward()
    assert torch.allclose(dq, qg.grad, atol=1e-11) and torch.allclose(dk, kg.grad, atol=1e-11)
    assert torch.allclose(dv, vg.grad, atol=1e-11) and torch.allclose(lse, lseg, atol=1e-11)
    # rounding points switched on with an identity rounding change nothing
    _, _, dq3, dk3, dv3 = orc.selected_attention_grads_ref(q, k, v, topk, 8, cu, do, dtype=torch.float64,
                                                           round_dtype=torch.float64)
    assert torch.equal(dq3, dq) and torch.equal(dk3, dk) and torch.equal(dv3, dv)

    def loss(q_, k_, v_):
        return float((orc.selected_attention_ref(q_, k_, v_, topk, 8, cu, dtype=torch.float64)[0] * do).sum())

    eps = 1e-6
    gen = torch.Generator().manual_seed(5)
    for name, x, gx in (("q", q, dq), ("k", k, dk), ("v", v, dv)):
        for _ in range(6):
            idx = tuple(int(torch.randint(0, s, (1,), generator=gen)) for s in x.shape)
            xp, xm = x.clone(), x.clone()
            xp[idx] += eps
            xm[idx] -= eps
            args_p = {"q": q, "k": k, "v": v}
            args_m = dict(args_p)
            args_p[name], args_m[name] = xp, xm
            fd = (loss(**{a + "_": b for a, b in args_p.items()}) -
                  loss(**{a + "_": b for a, b in args_m.items()})) / (2 * eps)
            assert abs(fd - float(gx[idx])) < 1e-6, (name, idx, fd, float(gx[idx]))


def test_gqa_dk_is_head_sum_of_expanded_keys():
    # dK over a group equals the sum over heads of the gradient w.r.t. GQA-expanded keys
    cu, q, k, v, do, topk = _case(n=64, hq=4, hkv=2, d=8, bk=8, t=3)
    _, _, _, dk, dv = orc.selected_attention_grads_ref(q, k, v, topk, 8, cu, do, dtype=torch.float64)
    kx = k.repeat_interleave(2, dim=1).clone().requires_grad_(True)
    vx = v.repeat_interleave(2, dim=1).clone().requires_grad_(True)
    topk_x = topk.repeat_interleave(2, dim=0)
    o, _ = orc.selected_attention_ref(q, kx, vx, topk_x, 8, cu, dtype=torch.float64)
    (o * do).sum().backward()
    assert torch.allclose(dk, kx.grad.reshape(64, 2, 2, 8).sum(2), atol=1e-11)
    assert torch.allclose(dv, vx.grad.reshape(64, 2, 2, 8).sum(2), atol=1e-11)


def _brute_index(topk, cu, bk):
    hkv, n, t = topk.shape
    nblk = [(cu[i + 1] - cu[i] + bk - 1) // bk for i in range(len(cu) - 1)]
    cub = [0]
    for x in nblk:
        cub.append(cub[-1] + x)
    out = []
    for h in range(hkv):
        pairs = []
        for s in range(len(cu) - 1):
            for i in range(cu[s], cu[s + 1]):
                for tt in range(t):
                    b = int(topk[h, i, tt])
                    if 0 <= b < nblk[s]:
                        pairs.append((cub[s] + b, i, tt))
        pairs.sort()
        out.append(pairs)
    return cub, out


@pytest.mark.parametrize("cu", [[0, 200], [0, 50, 51, 130, 200]])
def test_index_ref_against_brute_force(cu):
    bk, t = 16, 4
    topk = make_topk_idx(cu, 2, bk, t, seed=3)
    topk[1, 7, 2] = 99  # out-of-range id is ignored like padding
    cu_blocks, counts, starts, sel_tokens, slot_of = orc.build_index_ref(topk, cu, bk)
    cub, brute = _brute_index(topk, cu, bk)
    assert list(cu_blocks) == cub
    for h in range(2):
        pairs = brute[h]
        nb = cub[-1]
        bc = torch.bincount(torch.tensor([p[0] for p in pairs]), minlength=nb).numpy()
        assert np.array_equal(counts[h], bc)
        assert np.array_equal(starts[h, 1:], np.cumsum(bc)) and starts[h, 0] == 0
        assert list(sel_tokens[h, : len(pairs)]) == [p[1] for p in pairs]
        assert (sel_tokens[h, len(pairs):] == -1).all()
        for pos, (gb, i, tt) in enumerate(pairs):
            assert slot_of[h, i, tt] == pos
        assert (slot_of[h] >= 0).sum() == len(pairs)
        # ascending query id inside each block
        for gb in range(nb):
            seg = sel_tokens[h, starts[h, gb]: starts[h, gb + 1]]
            assert (np.diff(seg) > 0).all()


def test_synthetic_index_matches_stated_counts():
    # pair counts quoted for the 64K benchmark shape are reproduced at a size that runs fast
    cu = [0, 4096]
    topk = make_topk_idx(cu, 4, 64, 16, seed=0)
    pairs, keys = orc.count_pairs(topk, 64, cu)
    assert pairs == 4 * 57856 and keys == 4 * 3573760
    own = torch.arange(4096) // 64
    assert (topk[:, :, 0] == 0).all()
    assert ((topk == own[None, :, None]).sum(-1) == 1).all()
    valid = topk >= 0
    assert (valid.sum(-1) == torch.minimum(own + 1, torch.tensor(16))[None]).all()
    srt = torch.where(valid, topk, torch.full_like(topk, 10**6)).sort(-1).values
    assert (torch.where(valid, topk, torch.full_like(topk, 10**6)) == srt).all()


def test_rows_ref_equals_chunked_oracle():
    """The per-row sampler (explicit key lists) and the chunked oracle (block views, batched gathers) agree on every
    row and on the dK/dV of every block of a small ragged batch."""
    from synth_inputs import make_qkv, make_topk_idx
    cu = [0, 150, 150, 391]
    n, hq, hkv, d, bk, t = cu[-1], 4, 2, 32, 16, 4
    q, k, v, do = make_qkv(n, hq, hkv, d, torch.float32, seed=5)
    idx = make_topk_idx(cu, hkv, bk, t, seed=6)
    o, lse, dq, dk, dv = orc.selected_attention_grads_ref(q, k, v, idx, bk, cu, do, dtype=torch.float64)
    rows = list(range(n))
    for kh, first in [(0, 0), (1, 150 + 3 * bk), (1, 150 + 15 * bk), (0, 9 * bk)]:
        r = orc.selected_attention_rows_ref(q, k, v, idx, bk, cu, rows, do=do, key_block=(kh, first))
        assert torch.allclose(r["o"], o, atol=1e-10) and torch.allclose(r["lse"], lse, atol=1e-10)
        assert torch.allclose(r["dq"], dq, atol=1e-10)
        hi = min(first + bk, 150 if first < 150 else n)
        assert torch.allclose(r["dk_block"][: hi - first], dk[first:hi, kh], atol=1e-9)
        assert torch.allclose(r["dv_block"][: hi - first], dv[first:hi, kh], atol=1e-9)


def test_key_block_grads_ref_equals_other_oracles():
    """The vectorised per-block dK / dV (used for blocks that every query selects) equals the chunked oracle's
    slices and the per-row sampler, with and without the kernels' rounding points, including a block cut by the
    sequence end and a stored (perturbed) O / LSE as inputs."""
    from synth_inputs import make_qkv, make_topk_idx
    cu = [0, 150, 150, 391]
    n, hq, hkv, d, bk, t = cu[-1], 4, 2, 32, 16, 4
    q, k, v, do = make_qkv(n, hq, hkv, d, torch.float32, seed=15)
    idx = make_topk_idx(cu, hkv, bk, t, seed=16)
    o, lse, _, dk, dv = orc.selected_attention_grads_ref(q, k, v, idx, bk, cu, do, dtype=torch.float64)
    _, _, starts, sel_tokens, _ = orc.build_index_ref(idx, cu, bk)
    cases = [(0, 0, 0, 150), (1, 150, 10, 391), (1, 150 + 15 * bk, 25, 391), (0, 9 * bk, 9, 150)]
    for kh, first, gb, seq_end in cases:
        users = sel_tokens[kh, int(starts[kh, gb]):int(starts[kh, gb + 1])].tolist()
        assert users, "block without users"
        dk_b, dv_b = orc.key_block_grads_ref(q, k, v, do, o, lse, kh, first, users, bk, seq_end, chunk=37)
        hi = min(first + bk, seq_end)
        assert torch.allclose(dk_b[: hi - first], dk[first:hi, kh], atol=1e-9)
        assert torch.allclose(dv_b[: hi - first], dv[first:hi, kh], atol=1e-9)
        assert (dk_b[hi - first:] == 0).all() and (dv_b[hi - first:] == 0).all()
        # stored, perturbed forward results as inputs + bf16 rounding points: against the per-row sampler
        o_in = (o + 0.01 * torch.sin(torch.arange(o.numel(), dtype=torch.float64)).view_as(o))
        lse_in = lse + 0.003
        r = orc.selected_attention_rows_ref(q, k, v, idx, bk, cu, users, do=do, o_in=o_in, lse_in=lse_in,
                                            round_dtype=torch.bfloat16, key_block=(kh, first))
        dk_b, dv_b = orc.key_block_grads_ref(q, k, v, do, o_in, lse_in, kh, first, users, bk, seq_end,
                                             round_dtype=torch.bfloat16)
        assert torch.allclose(dk_b, r["dk_block"], atol=1e-9) and torch.allclose(dv_b, r["dv_block"], atol=1e-9)
