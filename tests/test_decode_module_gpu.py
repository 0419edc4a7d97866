"""GPU: the decode modules (fsa_preview.module) against the prefill layer.

N decode steps from a prefilled cache must give what `FlashSparseAttention` computes for the same tokens at the end
of the same sequence (y relative error within the layer tolerance of 2e-2).  Two regimes: few blocks (every block is
selected, and a compression window completes on the way) and many blocks (top-8 of ~48; the decode step ranks
bf16-rounded block scores as the prefill selection does, so it picks the same blocks).
"""
import math

import pytest
import torch

from fsa.module.fsa import FlashSparseAttention, RopeConfig
from fsa.ops import FSA_topk_sparse_attention
from fsa_hip import ops
from fsa_preview.module import FlashSparseAttentionDecode, FlashSparseAttentionDecodeKernel
from nsa_ref.ops import compressed_attention, linear_compress

pytestmark = pytest.mark.gpu

CFG = dict(hidden_size=1024, num_q_heads=8, num_kv_heads=2, head_dim=128, kernel_size=32, kernel_stride=16,
           block_size=64, topk=8, init_blocks=1, local_blocks=2, window_size=128)


def _rel(a, b):
    return ((a.float() - b.float()).norm() / b.float().norm()).item()


def _prefill_caches(layer, x, L):
    dev = x.device
    cu = torch.tensor([0, L], dtype=torch.int32, device=dev)
    k = layer.proj_k(x[:L]).view(L, layer.num_kv_heads, layer.head_dim)
    v = layer.proj_v(x[:L]).view(L, layer.num_kv_heads, layer.head_dim)
    ck, _ = linear_compress(k, layer.compress_key, cu, layer.kernel_size, layer.kernel_stride, layer.intra_block_pe)
    cv, _ = linear_compress(v, layer.compress_value, cu, layer.kernel_size, layer.kernel_stride, None)
    return k, v, ck, cv


@pytest.mark.parametrize("L,n_steps,min_ok", [(32 + 16 * 20 - 2, 20, 20), (3054, 24, 24)])
def test_decode_layer_steps_equal_prefill_rows(dev, L, n_steps, min_ok):
    print(f"case L={L} steps={n_steps}", flush=True)
    torch.manual_seed(5)
    layer = FlashSparseAttention(**CFG, rope_config=RopeConfig(head_dim=128)).to(dev).to(torch.bfloat16)
    dec = FlashSparseAttentionDecode(**CFG, rope_config=RopeConfig(head_dim=128)).to(dev).to(torch.bfloat16)
    dec.load_state_dict(layer.state_dict())
    n = L + n_steps
    x = torch.randn(n, CFG["hidden_size"], device=dev, dtype=torch.bfloat16)
    with torch.no_grad():
        y_ref = layer(x, torch.tensor([0, n], dtype=torch.int32, device=dev))
        k_c, v_c, ck_c, cv_c = _prefill_caches(layer, x, L)
    cu_q = torch.tensor([0, 1], dtype=torch.int32, device=dev)
    n_new_windows, errs = 0, []
    for t in range(n_steps):
        cu_k = torch.tensor([0, L + t + 1], dtype=torch.int32, device=dev)
        y, (k_new, v_new, ck_new, cv_new) = dec(x[L + t:L + t + 1], cu_q, cu_k, k_c, v_c, ck_c, cv_c,
                                                return_new_rows=True)
        assert y.shape == (1, CFG["hidden_size"]) and torch.isfinite(y.float()).all()
        errs.append(_rel(y[0], y_ref[L + t]))
        k_c, v_c = torch.cat([k_c, k_new]), torch.cat([v_c, v_new])
        if ck_new is not None:
            n_new_windows += 1
            ck_c, cv_c = torch.cat([ck_c, ck_new]), torch.cat([cv_c, cv_new])
    torch.cuda.synchronize()
    print("  rel errors per step: " + " ".join(f"{e:.1e}" for e in errs), flush=True)
    assert n_new_windows >= 1, "no compression window completed during the steps"
    # the caches grown step by step equal the prefill of the whole sequence
    with torch.no_grad():
        k_f, v_f, ck_f, cv_f = _prefill_caches(layer, x, n)
    # (up to the last bit: a projection of one row and of the whole sequence may run different GEMM kernels)
    def close(a, b):
        return a.shape == b.shape and (a.float() - b.float()).abs().max().item() <= 2.0 ** -6 * b.float().abs().max().item()
    assert close(k_c, k_f) and close(v_c, v_f) and close(ck_c, ck_f) and close(cv_c, cv_f)
    assert sum(e < 2e-2 for e in errs) >= min_ok, errs
    assert sorted(errs)[len(errs) // 2] < 1e-2


def test_decode_kernel_module_equals_prefill_ops(dev):
    """The kernel-level module (q / k / v given, no projections, no rotary) against the prefill operators on the same
    rows: compressed attention + selection, selected attention, band attention, gated sum for the last token."""
    torch.manual_seed(6)
    cfg = dict(CFG)
    hq, hkv, d, ks, st, bk, topk, win = 8, 2, 128, 32, 16, 64, 8, 128
    L = 700
    dtype = torch.bfloat16
    mod = FlashSparseAttentionDecodeKernel(**cfg).to(dev).to(dtype)
    for p in mod.parameters():
        torch.nn.init.normal_(p, std=0.02)
    q = torch.randn(L + 1, hq, d, device=dev, dtype=dtype)
    k = torch.randn(L + 1, hkv, d, device=dev, dtype=dtype)
    v = torch.randn(L + 1, hkv, d, device=dev, dtype=dtype)
    cu = torch.tensor([0, L + 1], dtype=torch.int32, device=dev)
    cu_prev = torch.tensor([0, L], dtype=torch.int32, device=dev)
    with torch.no_grad():
        ck_prev, _ = linear_compress(k[:L], mod.compress_key, cu_prev, ks, st, mod.intra_block_pe)
        cv_prev, _ = linear_compress(v[:L], mod.compress_value, cu_prev, ks, st, None)
        ck, cu_ck = linear_compress(k, mod.compress_key, cu, ks, st, mod.intra_block_pe)
        cv, _ = linear_compress(v, mod.compress_value, cu, ks, st, None)
        o_c, idx = compressed_attention(q, ck, cv, ks, st, bk, topk, cu, cu_ck, L + 1, ck.shape[0], None, 1, 2,
                                        parallel_topk_compute=False)
        o_s = FSA_topk_sparse_attention(q, k, v, idx, bk, cu)
        o_w, _ = ops.winattn_fwd(q, k, v, cu, L + 1, win)
        gate = mod.gate(q[L:].reshape(1, -1))
        want = (gate[:, 0:1] * o_c[L:].reshape(1, -1).float() + gate[:, 1:2] * o_s[L:].reshape(1, -1).float()
                + gate[:, 2:3] * o_w[L:].reshape(1, -1).float())
        got = mod(q[L:], k[L:], v[L:], torch.tensor([0, 1], dtype=torch.int32, device=dev), cu, k[:L], v[:L],
                  ck_prev, cv_prev)
        lit = mod(q[L:], k[L:], v[L:], torch.tensor([0, 1], dtype=torch.int32, device=dev), cu, k[:L], v[:L],
                  ck_prev, cv_prev, as_written=True)
    torch.cuda.synchronize()
    assert got.shape == (1, hq * d)
    err = (got.float() - want).abs().max().item()
    print(f"  kernel module vs prefill operators: max-abs {err:.3e}", flush=True)
    assert err <= 2e-2
    assert lit.shape == got.shape and torch.isfinite(lit.float()).all()
