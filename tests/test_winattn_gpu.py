"""GPU parity: sliding-window attention forward / backward vs the CPU oracle.
Tolerances as for selected attention (O, grads 2e-2 bf16 / 5e-3 fp16 plus one output ulp; LSE 1e-3)."""
import pytest
import torch

from fsa_hip import ops
from oracle import module as orc

pytestmark = pytest.mark.gpu
TOL = {torch.bfloat16: 2e-2, torch.float16: 5e-3}
ULP = {torch.bfloat16: 2.0 ** -8, torch.float16: 2.0 ** -11}

CASES = [
    ([0, 2048], 8, 2, 128, 512, torch.bfloat16),
    ([0, 20, 700, 701, 2100, 3000], 4, 4, 128, 512, torch.bfloat16),
    ([0, 1500], 6, 2, 64, 100, torch.float16),
    ([0, 1024], 4, 2, 256, 64, torch.float16),
    ([0, 300], 4, 1, 128, 1000, torch.bfloat16),   # window longer than the sequence: plain causal
]


@pytest.mark.parametrize("cu,hq,hkv,d,window,dtype", CASES)
def test_winattn_fwd_bwd(dev, cu, hq, hkv, d, window, dtype):
    print(f"case cu={cu} hq={hq} hkv={hkv} d={d} window={window} {dtype}", flush=True)
    gen = torch.Generator().manual_seed(31)
    n = cu[-1]
    std = 0.5 if d == 256 else 1.0
    q, k, v, do = ((torch.randn(n, h, d, generator=gen) * std).to(dtype) for h in (hq, hkv, hkv, hq))
    cu_t = torch.tensor(cu, dtype=torch.int32, device=dev)
    max_len = max(b - a for a, b in zip(cu[:-1], cu[1:]))
    qd, kd, vd, dod = (x.to(dev) for x in (q, k, v, do))
    o, lse = ops.winattn_fwd(qd, kd, vd, cu_t, max_len, window)
    dq, dk, dv = ops.winattn_bwd(qd, kd, vd, o, dod, lse, cu_t, max_len, window)
    torch.cuda.synchronize()
    qr, kr, vr = (x.float().requires_grad_(True) for x in (q, k, v))
    o_r, lse_r = orc.window_attention_ref(qr, kr, vr, cu, window)
    # the backward operator takes the stored (rounded) forward output: use it for the upstream product
    (o_r * do.float()).sum().backward()
    err_l = (lse.cpu() - lse_r.detach()).abs().max().item()
    assert err_l <= 1e-3
    for name, got, ref in (("o", o, o_r.detach()), ("dq", dq, qr.grad), ("dk", dk, kr.grad), ("dv", dv, vr.grad)):
        got = got.float().cpu()
        assert torch.isfinite(got).all(), name
        err = (got - ref).abs().max().item()
        excess = ((got - ref).abs() - ULP[dtype] * ref.abs()).max().item()
        rel = ((got - ref).norm() / ref.norm()).item()
        print(f"  {name}: max abs {err:.3e} (ref max {ref.abs().max().item():.2f}), rel Frobenius {rel:.2e}", flush=True)
        assert rel < 1e-2, name
        assert excess <= 2 * TOL[dtype], (name, err)
