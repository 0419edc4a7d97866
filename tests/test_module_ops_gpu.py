"""GPU parity: rotary embedding and linear compression (forward / backward) vs the CPU oracle."""
import math

import pytest
import torch

from fsa_hip import ops
from oracle import cmpattn as pre
from oracle import module as orc

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("start,stride", [(0, 1), (0, 16)])
@pytest.mark.parametrize("h,d", [(6, 128), (32, 128), (3, 64), (5, 256), (4, 96)])
def test_rope(dev, dtype, start, stride, h, d):
    gen = torch.Generator().manual_seed(41)
    cu = [0, 1000, 1001, 3000]
    x = torch.randn(3000, h, d, generator=gen).to(dtype)
    inv = orc.llama3_inv_freq(d, 500000.0)
    cu_t = torch.tensor(cu, dtype=torch.int32, device=dev)
    y = ops.rope(x.to(dev), cu_t, inv.to(dev), 1.0, start, stride)
    back = ops.rope(y, cu_t, inv.to(dev), 1.0, start, stride, inverse=True)
    torch.cuda.synchronize()
    ref = orc.rope_ref(x, cu, inv, start, stride, table_dtype=dtype)
    ulp = 2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -11
    # identical arithmetic up to the rounding of cos/sin (one table ulp on a few entries) and of the output
    err = (y.float().cpu() - ref).abs()
    assert (err <= 3 * ulp * ref.abs() + 4 * ulp).all(), err.max()
    assert (err > ulp * ref.abs() + 1e-6).float().mean().item() < 0.02
    err_b = (back.float().cpu() - x.float()).abs().max().item()
    assert err_b <= 8 * ulp * 4


CASES = [
    # cu_seqlens, H, D, ks, stride, dtype, with pe
    ([0, 2048], 4, 128, 32, 16, torch.bfloat16, True),
    ([0, 20, 700, 731, 2100, 3000], 2, 128, 32, 16, torch.bfloat16, True),
    ([0, 1500], 2, 128, 32, 16, torch.float16, False),
    ([0, 1100], 2, 256, 32, 16, torch.float16, True),
]


@pytest.mark.parametrize("cu,h,d,ks,st,dtype,with_pe", CASES)
def test_linear_compress_fwd_bwd(dev, cu, h, d, ks, st, dtype, with_pe):
    print(f"case cu={cu} h={h} d={d} {dtype} pe={with_pe}", flush=True)
    gen = torch.Generator().manual_seed(43)
    n = cu[-1]
    x = torch.randn(n, h, d, generator=gen).to(dtype)
    w = (torch.randn(h, ks * d, d, generator=gen) * math.sqrt(6.0 / (ks * d + d))).to(dtype)
    pe = (torch.randn(h, ks, d, generator=gen) * 0.1).to(dtype) if with_pe else None
    cu_y = pre.compressed_lens(cu, ks, st)
    dy = torch.randn(cu_y[-1], h, d, generator=gen).to(dtype)
    cu_x_t = torch.tensor(cu, dtype=torch.int32, device=dev)
    cu_y_t = torch.tensor(cu_y, dtype=torch.int32, device=dev)
    max_x = max(b - a for a, b in zip(cu[:-1], cu[1:]))
    max_y = max(b - a for a, b in zip(cu_y[:-1], cu_y[1:]))
    xd, wd, dyd = x.to(dev), w.to(dev), dy.to(dev)
    ped = pe.to(dev) if with_pe else None
    y = ops.linear_compress_fwd(xd, wd, cu_x_t, cu_y_t, cu_y[-1], max_y, ks, st, ped)
    dx, dw, dpe = ops.linear_compress_bwd(xd, wd, dyd, cu_x_t, cu_y_t, max_x, ks, st, ped)
    torch.cuda.synchronize()
    xr, wr = x.float().requires_grad_(True), w.float().requires_grad_(True)
    per = pe.float().requires_grad_(True) if with_pe else None
    y_r, cu_y_r = pre.linear_compress_ref(xr, wr, cu, ks, st, per)
    assert cu_y_r == cu_y
    (y_r * dy.float()).sum().backward()
    pairs = [("y", y, y_r.detach()), ("dx", dx, xr.grad), ("dw", dw, wr.grad)]
    if with_pe:
        pairs.append(("dpe", dpe, per.grad))
    ulp = 2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -11
    for name, got, ref in pairs:
        got = got.float().cpu()
        assert torch.isfinite(got).all(), name
        rel = ((got - ref).norm() / ref.norm()).item()
        excess = ((got - ref).abs() - 2 * ulp * ref.abs()).max().item()
        print(f"  {name}: rel Frobenius {rel:.2e}, max abs {(got - ref).abs().max().item():.3e} "
              f"(ref max {ref.abs().max().item():.2f})", flush=True)
        assert rel < 3 * ulp, name
        assert excess <= (2e-2 if dtype == torch.bfloat16 else 5e-3), name


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_gate_merge(dev, dtype):
    """One-pass gate-weighted merge and its backward against the fp32 formulas (one output rounding)."""
    gen = torch.Generator().manual_seed(9)
    n, h, d = 1003, 6, 128
    a, b, c, w = (torch.randn(n, h, d, generator=gen).to(dtype) for _ in range(4))
    gate = torch.sigmoid(torch.randn(n, 3, generator=gen)).to(dtype)
    out = ops.gate_merge_fwd(a.to(dev), b.to(dev), c.to(dev), gate.to(dev))
    d_a, d_b, d_c, d_g = ops.gate_merge_bwd(w.to(dev), a.to(dev), b.to(dev), c.to(dev), gate.to(dev))
    torch.cuda.synchronize()
    g32 = gate.float()
    ref = g32[:, 0, None, None] * a.float() + g32[:, 1, None, None] * b.float() + g32[:, 2, None, None] * c.float()
    ulp = 2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -11
    assert ((out.float().cpu() - ref).abs() <= ulp * ref.abs() + 1e-6).all()   # fp32 sum (fused multiply-adds), one rounding
    for i, (got, x) in enumerate(((d_a, a), (d_b, b), (d_c, c))):
        assert torch.equal(got.cpu(), (g32[:, i, None, None] * w.float()).to(dtype))
        dg = (w.float() * x.float()).sum((1, 2))
        assert torch.allclose(d_g[:, i].float().cpu(), dg, rtol=2.0 ** -7 if dtype == torch.bfloat16 else 2.0 ** -10, atol=1e-2)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("d,dn", [(96, 128), (40, 64), (192, 256), (128, 96), (64, 40)])
def test_pad_head_dim_entry_point(dev, dtype, d, dn):
    """fsa_pad_head_dim through the C ABI: the leading columns copied bit for bit, the rest zero, on a strided
    source (a slice of a fused projection output) - what a caller with head_dim 96 / 192 runs before and after
    the kernels, which are built for 64 / 128 / 256 (fsa_native_head_dim names the size)."""
    from fsa_hip import _lib
    lib = _lib.load()
    assert [lib.fsa_native_head_dim(x) for x in (1, 40, 64, 65, 96, 128, 129, 192, 256, 257)] == \
        [64, 64, 64, 128, 128, 128, 256, 256, 256, -1]
    gen = torch.Generator().manual_seed(5)
    n, h = 777, 6
    big = torch.randn(n, h + 2, d + 8, generator=gen).to(dtype).to(dev)
    src = big[:, 1 : 1 + h, 4 : 4 + d]                     # strides (h + 2) * (d + 8), d + 8, 1; offset 8 bytes-aligned
    out = torch.full((n, h, dn), 7.0, dtype=dtype, device=dev)
    rc = lib.fsa_pad_head_dim(src.data_ptr(), src.stride(0), src.stride(1), d, out.data_ptr(), out.stride(0),
                              out.stride(1), dn, n, h, torch.cuda.current_stream(dev).cuda_stream)
    assert rc == 0, lib.fsa_last_error()
    torch.cuda.synchronize()
    m = min(d, dn)
    assert torch.equal(out[..., :m], src[..., :m])
    assert (out[..., m:] == 0).all()
    # the Python layer takes the same route
    assert torch.equal(ops._pad_d(src, dn) if dn > d else ops._cut_d(src, dn), out)
