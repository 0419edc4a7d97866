"""GPU parity over drawn configurations: ragged batches, GQA groups 1..8 (3 and 6 included), head dims 64 / 128,
block sizes 32 / 64 / 128, top-k 3..16, block lists in arbitrary slot order with padding anywhere.

Same bars as the fixed cases: index lists bit-exact, O max-abs 2e-2 (bf16) / 5e-3 (fp16), base-2 LSE 1e-3,
gradients within the same bound plus one ulp of the output dtype.
"""
import numpy as np
import pytest
import torch

from fsa_hip import ops
from synth_inputs import make_qkv, make_topk_idx
from oracle import selattn as orc

pytestmark = pytest.mark.gpu

O_TOL = {torch.bfloat16: 2e-2, torch.float16: 5e-3}
ULP = {torch.bfloat16: 2.0 ** -8, torch.float16: 2.0 ** -11}


def _draw(seed):
    rng = np.random.default_rng(seed)
    nseq = int(rng.integers(1, 5))
    lens = [int(rng.choice([1, 7, 63, 64, 65, 200, 777, 1500, 2600])) for _ in range(nseq)]
    if seed % 4 == 0:
        lens[0] = 3100                     # block 0 of this sequence is shared by several dK/dV work-groups
    cu = [0]
    for l in lens:
        cu.append(cu[-1] + l)
    hkv = int(rng.choice([1, 2, 3]))
    g = int(rng.choice([1, 2, 3, 4, 6, 8]))
    d = int(rng.choice([64, 128]))
    bk = int(rng.choice([32, 64, 128]))
    t = int(rng.choice([3, 5, 8, 16]))
    dtype = torch.bfloat16 if rng.integers(2) else torch.float16
    return cu, hkv * g, hkv, d, bk, t, dtype


def _scramble(topk, seed):
    """Slots of every query in a random order, and one in eight non-forced entries replaced by padding."""
    gen = torch.Generator().manual_seed(seed)
    hkv, n, t = topk.shape
    drop = (torch.rand(hkv, n, t, generator=gen) < 0.125) & (topk > 0)
    out = torch.where(drop, torch.full_like(topk, -1), topk)
    perm = torch.rand(hkv, n, t, generator=gen).argsort(-1)
    return torch.gather(out, 2, perm).contiguous()


@pytest.mark.parametrize("seed", list(range(12)))
def test_drawn_configuration(dev, seed):
    cu, hq, hkv, d, bk, t, dtype = _draw(seed)
    print(f"case seed={seed} cu={cu} hq={hq} hkv={hkv} d={d} bk={bk} t={t} {dtype}", flush=True)
    _check(dev, seed, cu, hq, hkv, d, bk, t, dtype)


@pytest.mark.parametrize("nseq,maxlen,hkv,g,d,bk,t,dtype", [
    (1200, 40, 2, 2, 128, 32, 4, torch.bfloat16),
    (2500, 5, 1, 16, 128, 32, 1, torch.float16),
    (300, 300, 2, 3, 256, 128, 2, torch.bfloat16),
])
def test_many_short_sequences(dev, nseq, maxlen, hkv, g, d, bk, t, dtype):
    """Batches of hundreds to thousands of sequences of 0 .. maxlen tokens (empty ones included): every sequence
    is shorter than a few blocks, so most blocks are partial and most selections are forced ones."""
    rng = np.random.default_rng(nseq)
    lens = rng.integers(0, maxlen + 1, size=nseq)
    lens[0] = max(int(lens[0]), 1)
    cu = [0] + np.cumsum(lens).tolist()
    print(f"case nseq={nseq} n={cu[-1]} hq={hkv * g} hkv={hkv} d={d} bk={bk} t={t} {dtype}", flush=True)
    _check(dev, nseq, cu, hkv * g, hkv, d, bk, t, dtype, both_index_paths=True)


def _unforced(topk, cu, bk, seed):
    """Lists in which the forced blocks are not a given: a third of the queries lose block 0, another third their
    own block, and every query past its first block holds the block before its own (the layer's local_blocks = 2
    layout) in place of one of its random picks."""
    gen = torch.Generator().manual_seed(seed)
    out = topk.clone()
    hkv, n, t = out.shape
    own = torch.cat([torch.arange(b - a) // bk for a, b in zip(cu[:-1], cu[1:])])[None, :, None]   # [1, N, 1]
    which = torch.randint(0, 3, (hkv, n, 1), generator=gen)
    has_prev = ((out == own - 1) & (own >= 1)).any(-1, keepdim=True)
    # own - 1 replaces the first entry that is neither block 0, the own block nor padding
    free = (out > 0) & (out != own) & (out != own - 1)
    first_free = free & (free.int().cumsum(-1) == 1)
    out = torch.where(first_free & ~has_prev & (own >= 2), (own - 1).expand_as(out).to(out.dtype), out)
    out = torch.where((which == 0) & (out == 0) & (own >= 1), torch.full_like(out, -1), out)       # no block 0
    out = torch.where((which == 1) & (out == own) & (own >= 1), torch.full_like(out, -1), out)     # no own block
    return out


@pytest.mark.parametrize("cu,hq,hkv,d,bk,t,dtype", [([0, 2100, 2164, 5000], 8, 2, 128, 64, 8, torch.bfloat16),
                                                    ([0, 3300], 4, 4, 128, 64, 16, torch.float16)])
def test_lists_without_forced_blocks(dev, cu, hq, hkv, d, bk, t, dtype):
    """Nothing in the operator assumes that a query selects block 0 or its own block, or that it does not select the
    block before its own: lists without them (and with own - 1 everywhere) against the same oracle."""
    print(f"case cu={cu} hq={hq} hkv={hkv} d={d} bk={bk} t={t} {dtype}", flush=True)
    topk = _unforced(make_topk_idx(cu, hkv, bk, t, seed=77), cu, bk, 78)
    own = torch.cat([torch.arange(b - a) // bk for a, b in zip(cu[:-1], cu[1:])])[None, :, None]
    late = (own >= 2).expand_as(topk)[..., 0]
    assert ((topk == 0).any(-1) | ~late).float().mean() < 0.8 and ((topk == own).any(-1) | ~late).float().mean() < 0.8
    assert ((topk == own - 1).any(-1) | ~late).all()
    _check(dev, 5, cu, hq, hkv, d, bk, t, dtype, topk=topk)


def _check(dev, seed, cu, hq, hkv, d, bk, t, dtype, both_index_paths=False, topk=None):
    n = cu[-1]
    std = 1.0 if dtype == torch.bfloat16 else 0.5
    q, k, v, do = make_qkv(n, hq, hkv, d, dtype, seed=100 + seed, std=std)
    if topk is None:
        topk = _scramble(make_topk_idx(cu, hkv, bk, t, seed=200 + seed), 300 + seed)
    cu_t = torch.tensor(cu, dtype=torch.int32)
    index = ops.build_index(topk.to(dev), cu_t.to(dev), bk)
    cu_blocks, counts, starts, sel_tokens, slot_of = orc.build_index_ref(topk, cu, bk)
    nb = int(cu_blocks[-1])
    assert np.array_equal(index.counts.cpu().numpy()[:, :nb], counts)
    assert np.array_equal(index.starts.cpu().numpy()[:, : nb + 1], starts)
    assert np.array_equal(index.sel_tokens.cpu().numpy(), sel_tokens)
    assert np.array_equal(index.slot_of.cpu().numpy(), slot_of)
    if both_index_paths:
        import os
        os.environ["FSA_INDEX_RADIX"] = "1"      # the general (radix sort) path must build the same lists
        try:
            other = ops.build_index(topk.to(dev), cu_t.to(dev), bk)
        finally:
            os.environ.pop("FSA_INDEX_RADIX")
        assert torch.equal(other.sel_tokens, index.sel_tokens) and torch.equal(other.slot_of, index.slot_of)
        assert torch.equal(other.starts, index.starts) and torch.equal(other.counts, index.counts)

    qd, kd, vd, dod = (x.to(dev) for x in (q, k, v, do))
    o, lse = ops.selattn_fwd(qd, kd, vd, index)
    dq, dk, dv = ops.selattn_bwd(qd, kd, vd, o, dod, lse, index)
    torch.cuda.synchronize()
    o_ref, lse_ref = orc.selected_attention_ref(q.float(), k.float(), v.float(), topk, bk, cu)
    lse_c = lse.cpu()
    dead = torch.isinf(lse_ref)
    assert torch.equal(torch.isinf(lse_c), dead)
    err_o = (o.float().cpu() - o_ref).abs().max().item()
    err_l = (lse_c[~dead] - lse_ref[~dead]).abs().max().item() if (~dead).any() else 0.0
    print(f"  max|dO|={err_o:.3e} max|dLSE|={err_l:.3e}", flush=True)
    assert err_o <= O_TOL[dtype] and err_l <= 1e-3
    _, _, dq_r, dk_r, dv_r = orc.selected_attention_grads_ref(q.float(), k.float(), v.float(), topk, bk, cu,
                                                              do.float(), round_dtype=dtype,
                                                              o_in=o.float().cpu(), lse_in=lse_c)
    for name, got, ref in (("dq", dq, dq_r), ("dk", dk, dk_r), ("dv", dv, dv_r)):
        got = got.float().cpu()
        assert torch.isfinite(got).all(), name
        excess = ((got - ref).abs() - ULP[dtype] * ref.abs()).max().item()
        print(f"  max|d{name}|={(got - ref).abs().max().item():.3e}", flush=True)
        assert excess <= O_TOL[dtype], name
