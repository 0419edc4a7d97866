"""GPU parity for block_size 256 through the reference-named operator.

The reference accepts block_size 256 (fsa/ops/FSA_topk_sparse_attention.py:926); this build runs it on the
128-key kernels after rewriting every selected block as its two halves.  Checked here: the rewritten lists are
bit-exact against a host restatement, O / LSE / gradients meet the same tolerances as the other block sizes
against the oracle evaluated at block_size 256, and the dictionaries of `permute_results` are built for 256.
"""
import numpy as np
import pytest
import torch

from fsa.ops.FSA_topk_sparse_attention import (FSA_topk_sparse_attention, _topk_sparse_attention_bwd_opt,
                                               _topk_sparse_attention_fwd_opt)
from fsa_hip import ops
from synth_inputs import make_qkv, make_topk_idx
from oracle import selattn as orc

pytestmark = pytest.mark.gpu

TOL = {torch.bfloat16: 2e-2, torch.float16: 5e-3}
ULP = {torch.bfloat16: 2.0 ** -8, torch.float16: 2.0 ** -11}

CASES = [
    # cu_seqlens, Hq, Hkv, D, T, dtype
    ([0, 4096], 4, 2, 128, 8, torch.bfloat16),
    ([0, 300, 301, 2500, 4000], 4, 2, 128, 4, torch.bfloat16),   # ragged, a one-token sequence, partial blocks
    ([0, 3000], 6, 2, 64, 4, torch.float16),                     # g = 3
]


def _split_ref(topk, cu, factor, sub):
    hkv, n, t = topk.shape
    out = np.full((hkv, n, t * factor), -1, dtype=np.int32)
    tk = topk.numpy()
    for a, b in zip(cu[:-1], cu[1:]):
        for tok in range(a, b):
            qpos = tok - a
            for j in range(factor):
                sb = tk[:, tok, :].astype(np.int64) * factor + j
                ok = (tk[:, tok, :] >= 0) & (sb * sub <= qpos)
                out[:, tok, j::factor] = np.where(ok, sb, -1)
    return out


@pytest.mark.parametrize("cu,hq,hkv,d,t,dtype", CASES)
def test_block256(dev, cu, hq, hkv, d, t, dtype):
    print(f"case cu={cu} hq={hq} hkv={hkv} d={d} t={t} {dtype}", flush=True)
    bk, n = 256, cu[-1]
    q, k, v, do = make_qkv(n, hq, hkv, d, dtype, seed=21, std=1.0 if dtype == torch.bfloat16 else 0.5)
    topk = make_topk_idx(cu, hkv, bk, t, seed=22)
    cu_t = torch.tensor(cu, dtype=torch.int32, device=dev)
    topk_d = topk.to(dev)
    split = ops.split_topk_blocks(topk_d, cu_t, bk, 2).cpu().numpy()
    assert np.array_equal(split, _split_ref(topk, cu, 2, 128))

    qd, kd, vd, dod = (x.to(dev) for x in (q, k, v, do))
    scale = 1.0 / d ** 0.5
    o, lse, perm = _topk_sparse_attention_fwd_opt(qd, kd, vd, topk_d, bk, cu_t, cu_t, n, n, scale)
    dq, dk, dv = _topk_sparse_attention_bwd_opt(o, dod, lse, qd, kd, vd, topk_d, bk, cu_t, cu_t, n, n, scale, perm)
    torch.cuda.synchronize()
    o_ref, lse_ref = orc.selected_attention_ref(q.float(), k.float(), v.float(), topk, bk, cu)
    err_o = (o.float().cpu() - o_ref).abs().max().item()
    err_l = (lse.cpu() - lse_ref).abs().max().item()
    print(f"  max|dO|={err_o:.3e} max|dLSE|={err_l:.3e}", flush=True)
    assert err_o <= TOL[dtype] and err_l <= 1e-3
    _, _, dq_r, dk_r, dv_r = orc.selected_attention_grads_ref(q.float(), k.float(), v.float(), topk, bk, cu,
                                                              do.float(), round_dtype=dtype,
                                                              o_in=o.float().cpu(), lse_in=lse.cpu())
    for name, got, ref in (("dq", dq, dq_r), ("dk", dk, dk_r), ("dv", dv, dv_r)):
        got = got.float().cpu()
        assert torch.isfinite(got).all(), name
        excess = ((got - ref).abs() - ULP[dtype] * ref.abs()).max().item()
        print(f"  max|d{name}|={(got - ref).abs().max().item():.3e}", flush=True)
        assert excess <= TOL[dtype], name

    # the per-sequence dictionaries describe the caller's blocks of 256 keys
    cu_blocks, counts, starts, sel_tokens, slot_of = orc.build_index_ref(topk, cu, bk)
    for s in range(len(cu) - 1):
        d_s = perm[s]
        nb = int(cu_blocks[s + 1] - cu_blocks[s])
        assert d_s["real_num_blocks"] == nb
        for h in range(hkv):
            lo, hi = int(starts[h, cu_blocks[s]]), int(starts[h, cu_blocks[s + 1]])
            assert np.array_equal(d_s["valid_topk_idx_permuted_tile"][h].cpu().numpy(), sel_tokens[h, lo:hi] - cu[s])
            assert np.array_equal(d_s["valid_lens"][h].cpu().numpy()[:nb], counts[h, cu_blocks[s]:cu_blocks[s + 1]])

    # autograd entry point gives the same output
    q2 = qd.clone().requires_grad_(True)
    o2 = FSA_topk_sparse_attention(q2, kd, vd, topk_d, bk, cu_t)
    o2.backward(dod)
    assert torch.equal(o2, o) and torch.equal(q2.grad, dq)
