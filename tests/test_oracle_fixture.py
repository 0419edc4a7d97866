"""The committed oracle fixture (tests/golden/selattn_small.npz, written by tests/golden/make_oracle_fixture.py).

The reference holds no golden vectors, so the fixture is the frozen output of this build's oracle on one small
ragged case: the CPU test catches drift of the oracle or of the seeded input generators, the GPU test checks the
HIP path against the same committed numbers (index lists bit-exact, O 2e-2, LSE 1e-3, gradients 2e-2 + 2 ulp)."""
import importlib.util
import os

import numpy as np
import pytest
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
FIX = os.path.join(HERE, "golden", "selattn_small.npz")


def _maker():
    spec = importlib.util.spec_from_file_location("make_oracle_fixture", os.path.join(HERE, "golden", "make_oracle_fixture.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def test_oracle_reproduces_the_committed_fixture():
    fix = np.load(FIX)
    now = _maker().compute()
    assert sorted(fix.files) == sorted(now)
    for name in fix.files:
        a, b = fix[name], now[name]
        assert a.shape == b.shape and a.dtype == b.dtype, name
        if a.dtype.kind in "iu":
            assert np.array_equal(a, b), name
        else:
            fin = np.isfinite(a)
            assert np.array_equal(fin, np.isfinite(b)), name
            assert np.allclose(a[fin], b[fin], rtol=1e-5, atol=1e-6), name


@pytest.mark.gpu
def test_hip_path_matches_the_committed_fixture(dev):
    from fsa_hip import ops
    mk = _maker()
    fix = np.load(FIX)
    bf = lambda name: torch.from_numpy(fix[name]).view(torch.bfloat16)
    q, k, v, do = (bf(n + "_bf16").to(dev) for n in ("q", "k", "v", "do"))
    topk = torch.from_numpy(fix["topk"])
    cu = torch.tensor(mk.CU, dtype=torch.int32, device=dev)
    index = ops.build_index(topk.to(dev), cu, mk.BK)
    o, lse = ops.selattn_fwd(q, k, v, index)
    dq, dk, dv = ops.selattn_bwd(q, k, v, o, do, lse, index)
    torch.cuda.synchronize()
    nb = int(fix["cu_blocks"][-1])
    assert np.array_equal(index.counts.cpu().numpy()[:, :nb], fix["counts"])
    assert np.array_equal(index.starts.cpu().numpy()[:, : nb + 1], fix["starts"])
    assert np.array_equal(index.sel_tokens.cpu().numpy(), fix["sel_tokens"])
    assert np.array_equal(index.slot_of.cpu().numpy(), fix["slot_of"])
    assert (o.float().cpu().numpy() - fix["o"]).__abs__().max() <= 2e-2
    fin = np.isfinite(fix["lse"])
    assert np.array_equal(np.isfinite(lse.cpu().numpy()), fin)
    assert np.abs(lse.cpu().numpy()[fin] - fix["lse"][fin]).max() <= 1e-3
    for name, got in (("dq", dq), ("dk", dk), ("dv", dv)):
        ref = fix[name]
        err = np.abs(got.float().cpu().numpy() - ref) - 2 * 2.0 ** -8 * np.abs(ref)
        assert err.max() <= 2e-2, name
