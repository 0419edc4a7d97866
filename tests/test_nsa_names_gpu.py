"""GPU: the NSA-named selected-attention forms next to the FSA-named ones.

Mirrors the call pattern of the reference's own comparison script
(test/test_FSA_optimized_sel_attn.py:142-237): `_topk_sparse_attention_fwd_opt` /
`_topk_sparse_attention_bwd_opt` (fsa.ops) against `_topk_sparse_attention_fwd` /
`_topk_sparse_attention_bwd` (nsa_ref.ops) on the same seeded inputs, including a
backward that is fed a random `o` as the script does (:198-201).  Both name sets
run the same kernels here, so they must agree bit for bit; the values are checked
against the CPU oracle (O max-abs 2e-2 bf16 / 5e-3 fp16, LSE 1e-3).  Also covers
the per-sequence dictionaries of `permute_results` at the common block size of 64
and `reorder_topk_idx`.
"""
import numpy as np
import pytest
import torch

from fsa.ops.FSA_topk_sparse_attention import (FSATopkSparseAttention, _topk_sparse_attention_bwd_opt,
                                               _topk_sparse_attention_fwd_opt)
from nsa_ref.ops.topk_sparse_attention import (TopkSparseAttention, _topk_sparse_attention_bwd,
                                               _topk_sparse_attention_fwd, reorder_topk_idx,
                                               topk_sparse_attention)
from oracle import selattn as orc
from synth_inputs import make_qkv, make_topk_idx

pytestmark = pytest.mark.gpu

TOL = {torch.bfloat16: 2e-2, torch.float16: 5e-3}

CASES = [
    # cu_seqlens, Hq, Hkv, D, B_K, T, dtype
    ([0, 2048], 8, 4, 128, 64, 16, torch.bfloat16),
    ([0, 700, 1500, 2048], 16, 4, 128, 64, 16, torch.bfloat16),
    ([0, 1024], 4, 2, 128, 128, 8, torch.float16),
]


@pytest.mark.parametrize("cu,hq,hkv,d,bk,t,dtype", CASES)
def test_fsa_and_nsa_functional_forms_agree(dev, cu, hq, hkv, d, bk, t, dtype):
    print(f"case cu={cu} hq={hq} hkv={hkv} d={d} bk={bk} t={t} {dtype}", flush=True)
    n = cu[-1]
    q, k, v, do = make_qkv(n, hq, hkv, d, dtype, seed=42)
    topk = make_topk_idx(cu, hkv, bk, t, seed=43)
    qd, kd, vd, dod, topk_d = (x.to(dev) for x in (q, k, v, do, topk))
    cu_t = torch.tensor(cu, dtype=torch.int32, device=dev)
    seqlen = max(b - a for a, b in zip(cu[:-1], cu[1:]))
    sm_scale = 1.0 / d ** 0.5
    causal = bool((topk_d == -1).sum().item() != 0)

    o_opt, lse_opt, permute_results = _topk_sparse_attention_fwd_opt(
        qd, kd, vd, topk_d, bk, cu_t, cu_t, seqlen, seqlen, sm_scale, causal=causal)
    o_ref, lse_ref = _topk_sparse_attention_fwd(qd, kd, vd, topk_d, bk, cu_t, cu_t, seqlen, seqlen, sm_scale)
    assert o_ref.shape == (n, hq, d) and lse_ref.shape == (hq, n) and lse_ref.dtype == torch.float32
    assert torch.equal(o_opt, o_ref) and torch.equal(lse_opt, lse_ref)
    o_cpu, lse_cpu = orc.selected_attention_ref(q.float(), k.float(), v.float(), topk, bk, cu)
    assert (o_ref.float().cpu() - o_cpu).abs().max().item() <= TOL[dtype]
    assert (lse_ref.cpu() - lse_cpu).abs().max().item() <= 1e-3

    # backward as the reference's script calls it: a random o, the lse of the forward
    o_rand = torch.randn(n, hq, d, generator=torch.Generator().manual_seed(5)).to(dtype).to(dev)
    g_opt = _topk_sparse_attention_bwd_opt(o_rand, dod, lse_opt, qd, kd, vd, topk_d, bk, cu_t, cu_t, seqlen, seqlen,
                                           sm_scale, permute_results)
    g_ref = _topk_sparse_attention_bwd(o_rand, dod, lse_ref, qd, kd, vd, topk_d, bk, cu_t, cu_t, seqlen, seqlen,
                                       sm_scale)
    torch.cuda.synchronize()
    assert len(g_ref) == 3
    for a, b, like in zip(g_opt, g_ref, (qd, kd, vd)):
        assert b.shape == like.shape and b.dtype == dtype
        assert torch.equal(a, b)

    # the per-sequence dictionaries at the kernels' own block size
    cu_blocks, counts, starts, sel_tokens, _ = orc.build_index_ref(topk, cu, bk)
    assert len(permute_results) == len(cu) - 1
    for s in range(len(cu) - 1):
        d_s = permute_results[s]
        nb = int(cu_blocks[s + 1] - cu_blocks[s])
        assert d_s["real_num_blocks"] == nb and d_s["num_blocks"] == max(nb, t)
        assert d_s["valid_lens_all"].shape == (hkv, max(nb, t))
        for h in range(hkv):
            lo, hi = int(starts[h, cu_blocks[s]]), int(starts[h, cu_blocks[s + 1]])
            cnt = counts[h, cu_blocks[s]:cu_blocks[s + 1]]
            assert np.array_equal(d_s["valid_topk_idx_permuted_tile"][h].cpu().numpy(), sel_tokens[h, lo:hi] - cu[s])
            assert np.array_equal(d_s["valid_lens"][h].cpu().numpy()[:nb], cnt)
            assert np.array_equal(d_s["valid_start_indices"][h].cpu().numpy()[:nb], np.cumsum(cnt) - cnt)
        gmax = counts[:, cu_blocks[s] + 1:cu_blocks[s + 1]].max() if nb > 1 else counts[:, cu_blocks[s]].max()
        assert int(d_s["global_max_valid_tokens"]) == int(gmax)


def test_autograd_functions_agree(dev):
    cu, hq, hkv, d, bk, t, dtype = [0, 900, 1536], 8, 2, 128, 64, 8, torch.bfloat16
    n = cu[-1]
    q, k, v, do = make_qkv(n, hq, hkv, d, dtype, seed=52)
    topk_d = make_topk_idx(cu, hkv, bk, t, seed=53).to(dev)
    cu_t = torch.tensor(cu, dtype=torch.int32, device=dev)
    outs = []
    for fn in (lambda a, b, c: TopkSparseAttention.apply(a, b, c, topk_d, bk, cu_t, cu_t, 900, 900, None),
               lambda a, b, c: FSATopkSparseAttention.apply(a, b, c, topk_d, bk, cu_t, cu_t, 900, 900, None),
               lambda a, b, c: topk_sparse_attention(a, b, c, topk_d, bk, cu_t)):
        qd, kd, vd = (x.to(dev).requires_grad_(True) for x in (q, k, v))
        o = fn(qd, kd, vd)
        o.backward(do.to(dev))
        outs.append((o.detach(), qd.grad, kd.grad, vd.grad))
    torch.cuda.synchronize()
    for other in outs[1:]:
        for a, b in zip(outs[0], other):
            assert torch.equal(a, b)
    with pytest.raises(AssertionError):
        TopkSparseAttention.apply(q.to(dev).float(), k.to(dev).float(), v.to(dev).float(), topk_d, bk, cu_t, cu_t,
                                  900, 900, None)


def test_reorder_topk_idx(dev):
    """Built the way the reference's backward builds its arguments (FSA_topk_sparse_attention.py:1765-1790); the
    result holds, per kv block, the same SET of sequence-local query ids as the brute-force index (the reference
    leaves the order inside a block to an unstable argsort; here it ascends)."""
    cu, hkv, bk, t = [0, 500, 501, 1300], 2, 64, 6
    topk = make_topk_idx(cu, hkv, bk, t, seed=63)
    topk_d = topk.to(dev)
    cu_t = torch.tensor(cu, dtype=torch.int32, device=dev)
    cu_blocks, counts, starts, sel_tokens, _ = orc.build_index_ref(topk, cu, bk)
    seqlens = cu_t[1:] - cu_t[:-1]
    seqblocks = torch.ceil(seqlens / bk).to(torch.int32)
    cu_seqblocks = torch.cat([torch.zeros(1, dtype=torch.int32, device=dev), torch.cumsum(seqblocks, 0)]).to(torch.int32)
    assert np.array_equal(cu_seqblocks.cpu().numpy(), cu_blocks)
    nb = int(cu_blocks[-1])
    topk_q_count = torch.from_numpy(counts[:, :nb].copy()).to(dev)
    cu_topk_q_count = torch.cat([torch.zeros(hkv, 1, dtype=torch.int32, device=dev),
                                 torch.cumsum(topk_q_count, -1)], -1).to(torch.int32)
    got = reorder_topk_idx(topk_d, cu_topk_q_count, cu_t, cu_seqblocks, bk).cpu().numpy()
    assert got.dtype == np.int32 and got.shape == (hkv, int(cu_topk_q_count[:, -1].max()))
    seq_of_block = np.searchsorted(cu_blocks, np.arange(nb), side="right") - 1
    for h in range(hkv):
        for gb in range(nb):
            lo, hi = int(cu_topk_q_count[h, gb]), int(cu_topk_q_count[h, gb + 1])
            want = sel_tokens[h, int(starts[h, gb]):int(starts[h, gb + 1])] - cu[seq_of_block[gb]]
            assert np.array_equal(got[h, lo:hi], want)
        assert (got[h, int(cu_topk_q_count[h, -1]):] == -1).all()
