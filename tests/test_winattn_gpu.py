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


@pytest.mark.parametrize("direction", ["rising", "falling"])
def test_winattn_drifting_scores(dev, direction):
    """Scores that grow (or fall) steadily along the keys: the forward kernel moves its reference maximum only
    when a row outgrows it by 2^8, so a rising ramp of about 6 octaves per 64-key tile makes it rescale the
    accumulators on some tiles and keep a stale maximum on the others; a falling ramp never rescales after the
    first tile.  Output, LSE and gradients must still match the oracle."""
    cu, hq, hkv, d, window, dtype = [0, 1500, 2600], 4, 2, 128, 512, torch.bfloat16
    print(f"case drifting scores {direction}", flush=True)
    gen = torch.Generator().manual_seed(47)
    n = cu[-1]
    unit = torch.randn(d, generator=gen)
    unit = unit / unit.norm()
    pos = torch.arange(n, dtype=torch.float32)
    ramp = pos if direction == "rising" else (n - pos)
    # q . k / sqrt(d) * log2(e) rises by about 0.1 per key
    amp = 0.1 * (d ** 0.5) / 1.4427
    k = (torch.randn(n, hkv, d, generator=gen) * 0.3 + (ramp * amp / 4.0)[:, None, None] * unit).to(dtype)
    q = (torch.randn(n, hq, d, generator=gen) * 0.3 + 4.0 * unit).to(dtype)
    v, do = ((torch.randn(n, h, d, generator=gen)).to(dtype) for h in (hkv, hq))
    cu_t = torch.tensor(cu, dtype=torch.int32, device=dev)
    max_len = max(b - a for a, b in zip(cu[:-1], cu[1:]))
    qd, kd, vd, dod = (x.to(dev) for x in (q, k, v, do))
    o, lse = ops.winattn_fwd(qd, kd, vd, cu_t, max_len, window)
    dq, dk, dv = ops.winattn_bwd(qd, kd, vd, o, dod, lse, cu_t, max_len, window)
    torch.cuda.synchronize()
    qr, kr, vr = (x.float().requires_grad_(True) for x in (q, k, v))
    o_r, lse_r = orc.window_attention_ref(qr, kr, vr, cu, window)
    (o_r * do.float()).sum().backward()
    spread = (lse_r.detach().max() - lse_r.detach().min()).item()
    print(f"  LSE spread over the rows {spread:.1f} (base 2)", flush=True)
    assert spread > 50
    err_l = ((lse.cpu() - lse_r.detach()).abs() / lse_r.detach().abs().clamp_min(1.0)).max().item()
    assert err_l <= 1e-3
    # dQ along `unit` is a sum of dS times the ramp, i.e. a large offset times the row sum of dS, which is zero
    # only before dS is rounded to 16 bits for the matrix unit: that component is ill-conditioned by construction
    # and left out of the comparison (the rest of dQ is checked)
    def off_ramp(x):
        return x - (x @ unit)[..., None] * unit

    for name, got, ref in (("o", o, o_r.detach()), ("dq", dq, qr.grad), ("dk", dk, kr.grad), ("dv", dv, vr.grad)):
        got = got.float().cpu()
        assert torch.isfinite(got).all(), name
        if name == "dq":
            got, ref = off_ramp(got), off_ramp(ref)
        rel = ((got - ref).norm() / ref.norm()).item()
        excess = ((got - ref).abs() - ULP[dtype] * ref.abs()).max().item()
        print(f"  {name}: rel Frobenius {rel:.2e}, max excess {excess:.3e}", flush=True)
        assert rel < 1e-2, name
        assert excess <= 2 * TOL[dtype] * max(1.0, ref.abs().max().item()), name
