"""GPU parity at the shape of the CPU-plumbing configuration, whole tensors, against the fp32 oracle.

One sequence S=4096, Hkv=Hq=4 (GQA 1), head_dim 128, B_K=64, T=16, q / k / v ~ N(0,1) from a seed, the synthetic
block lists (block 0, own block, 14 distinct earlier blocks).  The oracle works in fp32 on the values the kernels
receive (the bf16 / fp16 roundings of the draws); O and LSE of every query are compared (max-abs 2e-2 bf16, 5e-3
fp16; LSE 1e-3).

The gradients are compared with the UNROUNDED oracle that recomputes its own forward (no kernel output enters the
reference, no rounding point of the kernels is applied): element-wise |got - ref| <= tol + 2 ulp |ref| and a
relative Frobenius error.  The same independent check runs at two more shapes (GQA 4 ragged batch, fp16 D=256) and
on the whole tensors of the headline shape at GQA 1 (S=65536).
"""
import pytest
import torch

from fsa_hip import ops
from oracle import selattn as orc
from synth_inputs import make_qkv, make_topk_idx

pytestmark = pytest.mark.gpu

TOL = {torch.bfloat16: 2e-2, torch.float16: 5e-3}
ULP = {torch.bfloat16: 2.0 ** -8, torch.float16: 2.0 ** -11}
REL = {torch.bfloat16: 6e-3, torch.float16: 1e-3}

CASES = [
    # name, cu_seqlens, Hq, Hkv, D, B_K, T, dtype, std
    ("C0-bf16", [0, 4096], 4, 4, 128, 64, 16, torch.bfloat16, 1.0),
    ("C0-fp16", [0, 4096], 4, 4, 128, 64, 16, torch.float16, 1.0),
    ("gqa4-ragged", [0, 1100, 1101, 3000], 8, 2, 128, 64, 16, torch.bfloat16, 1.0),
    ("fp16-d256", [0, 2048], 4, 2, 256, 128, 8, torch.float16, 0.5),
    # the headline shape at GQA 1, every element of O, LSE, dQ, dK, dV (about a minute of oracle time on the host)
    ("C1-gqa1-whole", [0, 65536], 4, 4, 128, 64, 16, torch.bfloat16, 1.0),
]


@pytest.mark.parametrize("name,cu,hq,hkv,d,bk,t,dtype,std", CASES)
def test_whole_tensor_against_unrounded_oracle(dev, name, cu, hq, hkv, d, bk, t, dtype, std):
    print(f"case {name} cu={cu} hq={hq} hkv={hkv} d={d} bk={bk} t={t} {dtype}", flush=True)
    n = cu[-1]
    q, k, v, do = make_qkv(n, hq, hkv, d, dtype, seed=0, std=std)
    topk = make_topk_idx(cu, hkv, bk, t, seed=1)
    cu_t = torch.tensor(cu, dtype=torch.int32, device=dev)
    index = ops.build_index(topk.to(dev), cu_t, bk)
    qd, kd, vd, dod = (x.to(dev) for x in (q, k, v, do))
    o, lse = ops.selattn_fwd(qd, kd, vd, index)
    dq, dk, dv = ops.selattn_bwd(qd, kd, vd, o, dod, lse, index)
    torch.cuda.synchronize()
    print("  device done, oracle running", flush=True)
    torch.set_num_threads(max(torch.get_num_threads(), min(16, __import__("os").cpu_count() or 1)))
    o_r, lse_r, dq_r, dk_r, dv_r = orc.selected_attention_grads_ref(q.float(), k.float(), v.float(), topk, bk, cu,
                                                                   do.float())
    eo = (o.float().cpu() - o_r).abs().max().item()
    el = (lse.cpu() - lse_r).abs().max().item()
    assert eo <= TOL[dtype] and el <= 1e-3, (eo, el)
    errs = {}
    for nm, got, ref in (("dQ", dq, dq_r), ("dK", dk, dk_r), ("dV", dv, dv_r)):
        got = got.float().cpu()
        assert torch.isfinite(got).all(), nm
        errs[nm] = (got - ref).abs().max().item()
        excess = ((got - ref).abs() - 2 * ULP[dtype] * ref.abs()).max().item()
        rel = ((got - ref).norm() / ref.norm()).item()
        print(f"  {nm}: max-abs {errs[nm]:.3e} (|ref| max {ref.abs().max().item():.2f}), rel {rel:.2e}", flush=True)
        assert excess <= TOL[dtype], (nm, errs[nm], excess)
        assert rel <= REL[dtype], (nm, rel)
    print(f"MAXABS {name}: O {eo:.2e} LSE {el:.2e} dQ {errs['dQ']:.2e} dK {errs['dK']:.2e} dV {errs['dV']:.2e} "
          f"(whole tensors, unrounded fp32 oracle)", flush=True)
