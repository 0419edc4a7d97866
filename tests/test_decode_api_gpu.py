"""GPU: the reference-named decode wrappers (batch of one) reproduce the prefill path for the last
token - the property the reference's own decode test asserts for the compression step
(test/test_cmp_attn_decode.py:218-232, rtol 1e-4 / atol 1e-5 there)."""
import math

import pytest
import torch

from fsa_hip import ops
from fsa_preview.ops import _compressed_attention_decode, _linear_compress_decode, _topk_sparse_attention_decode
from nsa_ref.ops import compressed_attention, linear_compress
from fsa.ops import FSA_topk_sparse_attention

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("L", [1552, 1553])   # the new token does / does not complete a window
def test_decode_step_equals_prefill_last_token(dev, L):
    gen = torch.Generator().manual_seed(51)
    hq, hkv, d, ks, st, bk, t = 8, 2, 128, 32, 16, 64, 8
    dtype = torch.bfloat16
    q = torch.randn(L, hq, d, generator=gen).to(dtype).to(dev)
    k = torch.randn(L, hkv, d, generator=gen).to(dtype).to(dev)
    v = torch.randn(L, hkv, d, generator=gen).to(dtype).to(dev)
    wk = (torch.randn(hkv, ks * d, d, generator=gen) * 0.02).to(dtype).to(dev)
    pe = (torch.randn(hkv, ks, d, generator=gen) * 0.1).to(dtype).to(dev)
    cu = torch.tensor([0, L], dtype=torch.int32, device=dev)
    cu_prev = torch.tensor([0, L - 1], dtype=torch.int32, device=dev)
    # compression: prefill(L) == prefill(L - 1) + one decode step
    ck_full, cu_ck = linear_compress(k, wk, cu, ks, st, pe)
    ck_prev, _ = linear_compress(k[: L - 1], wk, cu_prev, ks, st, pe)
    new = _linear_compress_decode(k[L - 1:], wk, ks, st, pe, prev_total_len=L - 1, token_buffer=k[L - ks: L - 1])
    n_full, n_prev = ck_full.shape[0], ck_prev.shape[0]
    if n_full > n_prev:
        assert new is not None and torch.equal(new[0], ck_full[-1])
    else:
        assert new is None
    assert torch.equal(ck_full[:n_prev], ck_prev)
    cv_full, _ = linear_compress(v, wk, cu, ks, st, None)
    # compressed attention + selection for the last token
    o_p, idx_p = compressed_attention(q, ck_full, cv_full, ks, st, bk, t, cu, cu_ck, L, n_full, None, 1, 2,
                                      parallel_topk_compute=False)  # bf16-rounded scores, the layer's path
    cu_q1 = torch.tensor([0, 1], dtype=torch.int32, device=dev)
    o_d, idx_d = _compressed_attention_decode(q[L - 1:], ck_full, cv_full, ks, st, bk, t, cu_q1, cu_ck, 1, n_full,
                                              None, 1, 2, query_start_index=L - 1)
    torch.cuda.synchronize()
    assert (o_d.float() - o_p[L - 1:].float()).abs().max().item() <= 2e-2
    assert torch.equal(idx_d[:, 0].sort(-1).values, idx_p[:, L - 1].sort(-1).values)
    # selected attention for the last token
    o_sel_p = FSA_topk_sparse_attention(q, k, v, idx_p, bk, cu)
    o_sel_d = _topk_sparse_attention_decode(q[L - 1:], k, v, idx_d, bk, cu_q1, cu)
    torch.cuda.synchronize()
    assert (o_sel_d.float() - o_sel_p[L - 1:].float()).abs().max().item() <= 2e-2
    # the reference's literal behaviour: key 0 only
    o_w = _topk_sparse_attention_decode(q[L - 1:], k, v, idx_d, bk, cu_q1, cu, as_written=True)
    assert torch.equal(o_w[0], v[0].repeat_interleave(hq // hkv, dim=0))
