"""GPU: index build + selected attention forward + backward recorded into a HIP graph.

The library never allocates, synchronises or reads device data on the host, and no result depends on the order in
which work-groups finish (partials are merged in a fixed order, no atomics): two eager runs are bit-identical, and a
recorded step replayed with new values in the same buffers (new q / k / v / dO and a new block list) equals the eager
step on those values bit for bit.  The graph is replayed three times with eager work in between.
"""
import pytest
import torch

from fsa_hip import ops
from synth_inputs import make_qkv, make_topk_idx

pytestmark = pytest.mark.gpu


def test_step_graph_replays_equal_eager(dev):
    cu, hq, hkv, d, bk, t, dtype = [0, 1500, 1501, 4000], 8, 2, 128, 64, 8, torch.bfloat16
    n = cu[-1]
    cu_t = torch.tensor(cu, dtype=torch.int32, device=dev)
    q, k, v, do = (x.to(dev) for x in make_qkv(n, hq, hkv, d, dtype, seed=0))
    topk = make_topk_idx(cu, hkv, bk, t, seed=1).to(dev)

    def step():
        index = ops.build_index(topk, cu_t, bk)
        o, lse = ops.selattn_fwd(q, k, v, index)
        dq, dk, dv = ops.selattn_bwd(q, k, v, o, do, lse, index)
        return o, lse, dq, dk, dv

    first = [x.clone() for x in step()]
    again = step()
    torch.cuda.synchronize()
    for a, b in zip(first, again):
        assert torch.equal(a, b), "two eager runs differ"

    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()
    torch.cuda.current_stream().wait_stream(side)
    with torch.cuda.graph(graph):
        g_out = step()
    for rep in range(3):
        print(f"replay {rep}", flush=True)
        qn, kn, vn, don = (x.to(dev) for x in make_qkv(n, hq, hkv, d, dtype, seed=10 + rep))
        q.copy_(qn), k.copy_(kn), v.copy_(vn), do.copy_(don)
        topk.copy_(make_topk_idx(cu, hkv, bk, t, seed=20 + rep).to(dev))
        graph.replay()
        torch.cuda.synchronize()
        got = [x.clone() for x in g_out]
        want = step()
        torch.cuda.synchronize()
        for name, a, b in zip(("o", "lse", "dq", "dk", "dv"), got, want):
            assert torch.equal(a, b), f"replay {rep}: {name} differs from the eager step"
            assert torch.isfinite(a.float()).all() or name == "lse"
        assert not torch.equal(got[0], first[0])   # the replay really saw the new values
