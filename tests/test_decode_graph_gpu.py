"""GPU: one decode step of the three batched entry points recorded into a HIP graph.

The request lengths live in device arrays (cu_seqlens, positions), so a recorded step stays valid while the caches
grow: the graph is replayed three times with lengths advanced in place between the replays (and eager work of the
test in between), and every replay is compared with the eager result for the same lengths - compressed attention
output and LSE, selected block ids (bit-exact) and selected attention output.
"""
import math

import pytest
import torch

from fsa_hip import ops

pytestmark = pytest.mark.gpu


def test_decode_step_graph_replays_equal_eager(dev):
    hq, hkv, d, bk, t, ks, st = 8, 2, 128, 64, 8, 32, 16
    cap = [3000, 700, 1500, 4100]                  # capacity of each request's cache
    lens0 = [2500, 300, 1000, 3900]                # tokens at the first replay
    gen = torch.Generator().manual_seed(9)
    cu_k = [0]
    cu_ck = [0]
    for c in cap:
        cu_k.append(cu_k[-1] + c)
        cu_ck.append(cu_ck[-1] + (c - ks) // st + 1)
    nreq = len(cap)
    q = torch.randn(nreq, hq, d, generator=gen).to(torch.bfloat16).to(dev)
    kc, vc = (torch.randn(cu_k[-1], hkv, d, generator=gen).to(torch.bfloat16).to(dev) for _ in range(2))
    ck, cv = (torch.randn(cu_ck[-1], hkv, d, generator=gen).to(torch.bfloat16).to(dev) for _ in range(2))
    # request b owns a slot of cap[b] rows of the caches (cu arrays = slot boundaries); how many of them hold tokens
    # is said by device arrays: the query position (compressed keys seen) and the sequence length (raw keys)
    cu_k_t = torch.tensor(cu_k, dtype=torch.int32, device=dev)
    cu_ck_t = torch.tensor(cu_ck, dtype=torch.int32, device=dev)
    pos = torch.tensor([l - 1 for l in lens0], dtype=torch.int32, device=dev)
    seqlens = torch.tensor(lens0, dtype=torch.int32, device=dev)
    max_ck = max(b - a for a, b in zip(cu_ck[:-1], cu_ck[1:]))
    nblk_max = max(math.ceil(c / bk) for c in cap)
    scale = 1.0 / math.sqrt(d)

    def step():
        o_c, lse_c, raw = ops.decode_cmpattn(q, ck, cv, cu_ck_t, pos, ks, st, max_ck)
        idx = ops.decode_topk(raw, lse_c, cu_ck_t, pos, seqlens, hq, ks, st, bk, t, nblk_max, softmax_scale=scale)
        o_s, lse_s = ops.decode_selattn(q, kc, vc, cu_k_t, idx, bk, seqlens=seqlens)[:2]
        return o_c, lse_c, idx, o_s

    step()                                           # first calls outside the capture (one-time set-up of the library)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()
    torch.cuda.current_stream().wait_stream(side)
    with torch.cuda.graph(graph):
        g_out = step()
    for rep in range(3):
        print(f"replay {rep}: positions {pos.tolist()}", flush=True)
        graph.replay()
        torch.cuda.synchronize()
        got = [x.clone() for x in g_out]
        want = step()                                # eager, same lengths
        torch.cuda.synchronize()
        assert torch.equal(got[2], want[2]), "selected block ids"
        assert torch.equal(got[0], want[0]) and torch.equal(got[1], want[1]), "compressed attention"
        assert torch.equal(got[3], want[3]), "selected attention"
        assert torch.isfinite(got[0].float()).all() and torch.isfinite(got[3].float()).all()
        # slots with lengths == the same tokens packed back to back
        lens = seqlens.tolist()
        rows = torch.cat([torch.arange(cu_k[b], cu_k[b] + lens[b]) for b in range(nreq)]).to(dev)
        cu_packed = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32, device=dev)
        o_packed = ops.decode_selattn(q, kc[rows], vc[rows], cu_packed, want[2], bk)[0]
        torch.cuda.synchronize()
        assert (o_packed.float() - got[3].float()).abs().max().item() <= 1e-2, "slot lengths vs packed caches"
        pos += 37                                    # the caches grow between the replays
        seqlens += 37
        q.copy_(torch.randn(nreq, hq, d, generator=gen).to(torch.bfloat16))


def test_selected_decode_with_slot_lengths(dev):
    """`seqlens` cuts every request to its valid rows: equal to the packed caches; a request with no valid row gives
    a zero output row with LSE -inf; block ids past the valid rows are ignored."""
    hq, hkv, d, bk, t = 4, 2, 64, 32, 4
    cap = [300, 200, 500]
    lens = [257, 0, 31]
    gen = torch.Generator().manual_seed(4)
    cu = [0]
    for c in cap:
        cu.append(cu[-1] + c)
    q = torch.randn(3, hq, d, generator=gen).to(torch.float16).to(dev)
    kc, vc = (torch.randn(cu[-1], hkv, d, generator=gen).to(torch.float16).to(dev) for _ in range(2))
    idx = torch.tensor([[[0, 8, 3, 9], [0, 1, -1, -1], [0, 1, 2, -1]]] * hkv, dtype=torch.int32, device=dev)  # 9, 1, 2: past the rows
    cu_t = torch.tensor(cu, dtype=torch.int32, device=dev)
    sl = torch.tensor(lens, dtype=torch.int32, device=dev)
    o, lse = ops.decode_selattn(q, kc, vc, cu_t, idx, bk, seqlens=sl)
    rows = torch.cat([torch.arange(cu[b], cu[b] + lens[b]) for b in range(3)]).to(dev)
    cu_p = torch.tensor([0, 257, 257, 288], dtype=torch.int32, device=dev)
    o_p, lse_p = ops.decode_selattn(q, kc[rows], vc[rows], cu_p, idx, bk)
    torch.cuda.synchronize()
    assert torch.equal(o, o_p) and torch.equal(lse, lse_p)
    assert (o[1] == 0).all() and torch.isinf(lse[:, 1]).all() and (lse[:, 1] < 0).all()
    assert torch.isfinite(o.float()).all() and torch.isfinite(lse[:, [0, 2]]).all()
