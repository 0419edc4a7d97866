"""GPU: the allocation-free decode entry point `fsa_decode_selattn_static` against `fsa_decode_selattn`.

Same kernels and the same partial layout, so the results must be bit-identical.  Two calls in a row share the
library's built-in scratch buffer, the second with a smaller batch (stale partials of the first call stay behind
it in the buffer); sizes beyond the buffer are refused with a clear error and launch nothing.
"""
import pytest
import torch

from fsa_hip import _lib, ops

pytestmark = pytest.mark.gpu


def _inputs(lens, hq, hkv, d, bk, t, dtype, seed, dev):
    gen = torch.Generator().manual_seed(seed)
    b = len(lens)
    cu = [0]
    for l in lens:
        cu.append(cu[-1] + l)
    q = torch.randn(b, hq, d, generator=gen).to(dtype).to(dev)
    kc = torch.randn(cu[-1], hkv, d, generator=gen).to(dtype).to(dev)
    vc = torch.randn(cu[-1], hkv, d, generator=gen).to(dtype).to(dev)
    idx = torch.full((hkv, b, t), -1, dtype=torch.int32)
    for h in range(hkv):
        for i, l in enumerate(lens):
            nb = (l + bk - 1) // bk
            pick = torch.randperm(nb, generator=gen)[: min(t, nb)]
            idx[h, i, : pick.numel()] = pick.to(torch.int32)
    return q, kc, vc, torch.tensor(cu, dtype=torch.int32, device=dev), idx.to(dev)


def test_static_scratch_entry_point_matches_workspace_entry_point(dev):
    hq, hkv, d, bk, t, dtype = 8, 2, 128, 64, 16, torch.bfloat16
    gen = torch.Generator().manual_seed(91)
    first = torch.randint(40, 3000, (96,), generator=gen).tolist()     # many requests: shares cross pair boundaries
    second = [2500, 70, 1300]                                           # then a smaller call on the same buffer
    for n_call, lens in enumerate((first, second)):
        print(f"call {n_call}: {len(lens)} requests", flush=True)
        q, kc, vc, cu, idx = _inputs(lens, hq, hkv, d, bk, t, dtype, 92 + n_call, dev)
        o_ref, lse_ref = ops.decode_selattn(q, kc, vc, cu, idx, bk)
        o = torch.full((len(lens), hq, d), float("nan"), dtype=dtype, device=dev)
        lse = torch.full((hq, len(lens)), float("nan"), dtype=torch.float32, device=dev)
        ops.decode_selattn_static(q, kc, vc, cu, idx, bk, o, lse)
        torch.cuda.synchronize()
        assert torch.isfinite(o.float()).all() and torch.isfinite(lse).all()
        assert torch.equal(o, o_ref) and torch.equal(lse, lse_ref)


def test_static_scratch_rejects_sizes_beyond_the_buffer(dev):
    lib = _lib.load()
    hq, hkv, d, bk, t, dtype = 64, 8, 256, 64, 4, torch.bfloat16
    b = 8
    assert lib.fsa_decode_workspace_bytes(b, hq, hkv, d, 0) > (16 << 20)
    q, kc, vc, cu, idx = _inputs([100] * b, hq, hkv, d, bk, t, dtype, 95, dev)
    o = torch.zeros((b, hq, d), dtype=dtype, device=dev)
    lse = torch.zeros((hq, b), dtype=torch.float32, device=dev)
    with pytest.raises(ValueError, match="scratch"):
        ops.decode_selattn_static(q, kc, vc, cu, idx, bk, o, lse)
    torch.cuda.synchronize()
    assert (o == 0).all() and (lse == 0).all()
