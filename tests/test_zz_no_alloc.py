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


def test_static_scratch_call_can_be_recorded_into_a_graph(dev):
    """What the entry point exists for: the call allocates nothing, so it can be recorded into a HIP graph with
    caller-owned outputs.  After one eager call (buffer lookup), the call is captured and replayed on new query
    values, with eager work and synchronisations between the replays; every replay must equal the eager
    workspace entry point bit for bit.  An allocation inside the call would fail the capture."""
    hq, hkv, d, bk, t, dtype = 8, 2, 128, 64, 16, torch.bfloat16
    lens = [1500, 64, 700, 2999]
    q, kc, vc, cu, idx = _inputs(lens, hq, hkv, d, bk, t, dtype, 97, dev)
    o = torch.zeros((len(lens), hq, d), dtype=dtype, device=dev)
    lse = torch.zeros((hq, len(lens)), dtype=torch.float32, device=dev)
    ops.decode_selattn_static(q, kc, vc, cu, idx, bk, o, lse)          # eager first call: looks the buffer up
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        ops.decode_selattn_static(q, kc, vc, cu, idx, bk, o, lse)
    gen = torch.Generator().manual_seed(98)
    for rep in range(4):
        q.copy_(torch.randn(q.shape, generator=gen).to(dtype))
        o.fill_(float("nan"))
        lse.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        o_ref, lse_ref = ops.decode_selattn(q, kc, vc, cu, idx, bk)     # eager work between the replays
        torch.cuda.synchronize()
        assert torch.equal(o, o_ref) and torch.equal(lse, lse_ref), rep


def test_static_scratch_calls_on_two_streams_do_not_overlap(dev):
    """Consecutive eager calls on different streams share the one buffer: the second waits for the first's
    completion event inside the library, so both results are exact without any synchronisation by the caller."""
    hq, hkv, d, bk, t, dtype = 8, 2, 128, 64, 16, torch.bfloat16
    gen = torch.Generator().manual_seed(99)
    a_lens = torch.randint(500, 3000, (64,), generator=gen).tolist()
    b_lens = [2000, 100]
    ins_a = _inputs(a_lens, hq, hkv, d, bk, t, dtype, 100, dev)
    ins_b = _inputs(b_lens, hq, hkv, d, bk, t, dtype, 101, dev)
    ref_a = ops.decode_selattn(*ins_a, bk)
    ref_b = ops.decode_selattn(*ins_b, bk)
    outs = []
    for lens in (a_lens, b_lens):
        outs.append((torch.zeros((len(lens), hq, d), dtype=dtype, device=dev),
                     torch.zeros((hq, len(lens)), dtype=torch.float32, device=dev)))
    torch.cuda.synchronize()
    s1, s2 = torch.cuda.Stream(dev), torch.cuda.Stream(dev)
    for _ in range(3):
        with torch.cuda.stream(s1):
            ops.decode_selattn_static(*ins_a, bk, *outs[0])
        with torch.cuda.stream(s2):
            ops.decode_selattn_static(*ins_b, bk, *outs[1])
    torch.cuda.synchronize()
    assert torch.equal(outs[0][0], ref_a[0]) and torch.equal(outs[0][1], ref_a[1])
    assert torch.equal(outs[1][0], ref_b[0]) and torch.equal(outs[1][1], ref_b[1])
