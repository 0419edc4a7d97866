"""GPU parity: HIP selected-attention forward and index vs the CPU oracle.

Tolerances (from the task statement): O max-abs 2e-2 for bf16, 5e-3 for fp16;
base-2 LSE max-abs 1e-3; index lists bit-exact.
"""
import numpy as np
import pytest
import torch

from fsa_hip import ops
from synth_inputs import make_qkv, make_topk_idx
from oracle import selattn as orc

pytestmark = pytest.mark.gpu

O_TOL = {torch.bfloat16: 2e-2, torch.float16: 5e-3}
LSE_TOL = 1e-3


def _run_case(dev, cu, hq, hkv, d, bk, t, dtype, seed, std=1.0):
    n = cu[-1]
    q, k, v = make_qkv(n, hq, hkv, d, dtype, seed=seed, std=std, with_do=False)
    topk = make_topk_idx(cu, hkv, bk, t, seed=seed + 1)
    cu_t = torch.tensor(cu, dtype=torch.int32)
    index = ops.build_index(topk.to(dev), cu_t.to(dev), bk)
    o, lse = ops.selattn_fwd(q.to(dev), k.to(dev), v.to(dev), index)
    torch.cuda.synchronize()
    o_ref, lse_ref = orc.selected_attention_ref(q.float(), k.float(), v.float(), topk, bk, cu)
    return index, topk, o.float().cpu(), lse.cpu(), o_ref, lse_ref


def _check_index(index, topk, cu, bk):
    cu_blocks, counts, starts, sel_tokens, slot_of = orc.build_index_ref(topk, cu, bk)
    nb = int(cu_blocks[-1])
    assert np.array_equal(index.cu_blocks.cpu().numpy(), cu_blocks)
    got_counts = index.counts.cpu().numpy()
    assert np.array_equal(got_counts[:, :nb], counts)
    assert (got_counts[:, nb:] == 0).all()
    got_starts = index.starts.cpu().numpy()
    assert np.array_equal(got_starts[:, : nb + 1], starts)
    assert np.array_equal(index.sel_tokens.cpu().numpy(), sel_tokens)
    assert np.array_equal(index.slot_of.cpu().numpy(), slot_of)


CASES = [
    # cu_seqlens, Hq, Hkv, D, B_K, T, dtype
    ([0, 1024], 4, 4, 128, 64, 16, torch.bfloat16),
    ([0, 2048], 8, 4, 128, 64, 16, torch.bfloat16),
    ([0, 1536], 16, 4, 128, 64, 16, torch.bfloat16),
    ([0, 700, 701, 1900, 2048], 8, 2, 128, 64, 8, torch.bfloat16),   # ragged varlen, 1-token seq
    ([0, 1000], 6, 2, 128, 32, 4, torch.float16),                    # g = 3, partial last block
    ([0, 2048], 4, 2, 256, 128, 8, torch.float16),
    ([0, 512], 4, 1, 64, 64, 16, torch.bfloat16),                    # T > number of blocks
    ([0, 33], 2, 2, 128, 64, 16, torch.bfloat16),                    # shorter than one block
    # the remaining (head_dim, block size) pairs of the dispatch table
    ([0, 900], 4, 2, 128, 128, 4, torch.bfloat16),
    ([0, 700], 4, 2, 64, 32, 6, torch.bfloat16),
    ([0, 900], 2, 2, 64, 128, 4, torch.float16),
    ([0, 500], 4, 2, 256, 32, 6, torch.float16),
    ([0, 700], 2, 1, 256, 64, 6, torch.bfloat16),
    # head dims without a kernel of their own run zero-padded on the next size up (the reference takes any <= 256)
    ([0, 800], 4, 2, 96, 64, 8, torch.bfloat16),
    ([0, 600], 2, 1, 40, 32, 4, torch.float16),
    ([0, 500], 2, 2, 192, 64, 4, torch.bfloat16),
    ([0, 0, 300, 300, 1100, 1100], 16, 1, 128, 64, 8, torch.bfloat16),   # empty sequences, GQA group of 16
]


@pytest.mark.parametrize("cu,hq,hkv,d,bk,t,dtype", CASES)
def test_fwd_matches_oracle(dev, cu, hq, hkv, d, bk, t, dtype):
    print(f"case cu={cu} hq={hq} hkv={hkv} d={d} bk={bk} t={t} {dtype}", flush=True)
    std = 0.5 if d == 256 else 1.0
    index, topk, o, lse, o_ref, lse_ref = _run_case(dev, cu, hq, hkv, d, bk, t, dtype, seed=42, std=std)
    _check_index(index, topk, cu, bk)
    assert torch.isfinite(o).all() and torch.isfinite(lse).all()
    err_o = (o - o_ref).abs().max().item()
    err_l = (lse - lse_ref).abs().max().item()
    print(f"  max|dO|={err_o:.3e} max|dLSE|={err_l:.3e}", flush=True)
    assert err_o <= O_TOL[dtype]
    assert err_l <= LSE_TOL


INDEX_CASES = [
    # cu_seqlens, Hkv, B_K, T
    ([0, 5000], 2, 64, 16),
    ([0, 300, 301, 2500, 2500, 4000], 3, 32, 5),      # ragged, an empty and a one-token sequence, odd T
    ([0, 70000], 1, 16, 8),                          # 4375 blocks: beyond the counting path
    ([0, 9000], 2, 128, 24),                         # T not a power of two, partial last tile
]


@pytest.mark.parametrize("cu,hkv,bk,t", INDEX_CASES)
@pytest.mark.parametrize("radix", [False, True])
def test_index_both_paths(dev, monkeypatch, cu, hkv, bk, t, radix):
    """The counting path and the radix-sort path of the index build give the same, bit-exact lists."""
    print(f"case cu={cu} hkv={hkv} bk={bk} t={t} radix={radix}", flush=True)
    if radix:
        monkeypatch.setenv("FSA_INDEX_RADIX", "1")
    else:
        monkeypatch.delenv("FSA_INDEX_RADIX", raising=False)
    topk = make_topk_idx(cu, hkv, bk, t, seed=5)
    # a few out-of-range and padded entries in the middle of rows
    gen = torch.Generator().manual_seed(6)
    bad = torch.rand(topk.shape, generator=gen) < 0.02
    topk = torch.where(bad, torch.full_like(topk, -1), topk)
    cu_t = torch.tensor(cu, dtype=torch.int32)
    index = ops.build_index(topk.to(dev), cu_t.to(dev), bk)
    torch.cuda.synchronize()
    _check_index(index, topk, cu, bk)
