"""GPU parity at the full benchmark sizes, where the whole-tensor oracle would take minutes:

* index lists bit-exact against the CPU oracle (a sort of N*T keys, cheap at any size);
* O / LSE / dQ of a seeded SAMPLE of queries, and dK / dV of sampled key blocks, against the per-row oracle
  (same tolerances as the small cases: 2e-2 bf16, 5e-3 fp16, LSE 1e-3, plus one output ulp for gradients);
* dK / dV of block 0 - selected by every query, the one block whose rows are dealt to many work-groups and whose
  fp32 partials meet in the reduce kernel - element by element against the vectorised per-block oracle;
* size-independent identities over the WHOLE output:
    - scaling V by 2 scales O by exactly 2 and leaves LSE bit-identical (powers of two commute with rounding
      outside the subnormal range; bit-exact for bf16, one ulp for fp16);
    - sum_p dV[p, kh] = sum over the group's heads and all queries of dO   (rows of P sum to one);
    - sum <k, dK> = sum <q, dQ> per kv head   (both equal sum dS_ip s_ip / c: scale invariance of q.k).
  A dropped tile, a wrong block or a double-counted row breaks one of them.
"""
import math

import numpy as np
import pytest
import torch

from fsa_hip import ops
from synth_inputs import make_qkv, make_topk_idx
from oracle import selattn as orc

pytestmark = pytest.mark.gpu

TOL = {torch.bfloat16: 2e-2, torch.float16: 5e-3}
ULP = {torch.bfloat16: 2.0 ** -8, torch.float16: 2.0 ** -11}

CASES = [
    # name, S, Hq, Hkv, D, B_K, T, dtype, std
    ("C1-gqa4", 65536, 16, 4, 128, 64, 16, torch.bfloat16, 1.0),
    ("C1-gqa2", 65536, 8, 4, 128, 64, 16, torch.bfloat16, 1.0),
    ("C1-gqa1", 65536, 4, 4, 128, 64, 16, torch.bfloat16, 1.0),
    ("C3", 131072, 4, 2, 256, 128, 8, torch.float16, 0.5),
]


@pytest.mark.parametrize("name,n,hq,hkv,d,bk,t,dtype,std", CASES)
def test_selected_attention_full_size(dev, name, n, hq, hkv, d, bk, t, dtype, std):
    print(f"case {name} S={n} hq={hq} hkv={hkv} d={d} bk={bk} t={t} {dtype}", flush=True)
    g = hq // hkv
    cu = [0, n]
    q, k, v, do = make_qkv(n, hq, hkv, d, dtype, seed=11, std=std)
    topk = make_topk_idx(cu, hkv, bk, t, seed=12)
    cu_t = torch.tensor(cu, dtype=torch.int32, device=dev)
    index = ops.build_index(topk.to(dev), cu_t, bk)
    qd, kd, vd, dod = (x.to(dev) for x in (q, k, v, do))
    o, lse = ops.selattn_fwd(qd, kd, vd, index)
    dq, dk, dv = ops.selattn_bwd(qd, kd, vd, o, dod, lse, index)
    o2, lse2 = ops.selattn_fwd(qd, kd, vd * 2, index)
    torch.cuda.synchronize()

    # index: bit-exact
    cu_blocks, counts, starts, sel_tokens, slot_of = orc.build_index_ref(topk, cu, bk)
    nb = int(cu_blocks[-1])
    assert np.array_equal(index.cu_blocks.cpu().numpy(), cu_blocks)
    assert np.array_equal(index.counts.cpu().numpy()[:, :nb], counts)
    assert np.array_equal(index.starts.cpu().numpy()[:, : nb + 1], starts)
    assert np.array_equal(index.sel_tokens.cpu().numpy(), sel_tokens)
    assert np.array_equal(index.slot_of.cpu().numpy(), slot_of)

    # whole-output identities
    assert torch.isfinite(o.float()).all() and torch.isfinite(lse).all()
    assert torch.equal(lse2, lse)
    if dtype == torch.bfloat16:
        assert torch.equal(o2, o * 2)
    else:   # fp16 partial rows can be subnormal, where doubling no longer commutes with rounding: allow one ulp
        assert ((o2.float() - 2 * o.float()).abs() <= 2.0 ** -10 * o2.float().abs() + 2.0 ** -20).all()
    dof, dvf = dod.double(), dv.double()
    lhs = dvf.sum(0)                                               # [Hkv, D]
    rhs = dof.view(n, hkv, g, d).sum((0, 2))
    half_ulp = ULP[dtype] / 2
    walk = 6 * half_ulp * dvf.pow(2).sum(0).sqrt() + 1e-6          # random-walk bound of the output rounding
    print(f"  sum dV identity: max dev {(lhs - rhs).abs().max().item():.3e}, bound min {walk.min().item():.3e}", flush=True)
    assert ((lhs - rhs).abs() <= walk).all()
    kdk = (kd.double() * dk.double()).sum((0, 2))                  # [Hkv]
    qdq = (qd.double() * dq.double()).view(n, hkv, g, d).sum((0, 2, 3))
    scale_ = (kd.double() * dk.double()).abs().sum((0, 2))
    print(f"  <k,dK> vs <q,dQ>: {kdk.tolist()} vs {qdq.tolist()}", flush=True)
    assert ((kdk - qdq).abs() <= 4 * half_ulp * scale_ / math.sqrt(n) * 8 + 1e-3).all()

    # sampled queries
    gen = torch.Generator().manual_seed(13)
    rows = sorted(set([0, 1, bk - 1, bk, n - 1, n - bk] + torch.randint(0, n, (90,), generator=gen).tolist()))
    oc, lc = o.float().cpu(), lse.cpu()
    r = orc.selected_attention_rows_ref(q, k, v, topk, bk, cu, rows, do=do, o_in=oc, lse_in=lc, round_dtype=dtype)
    eo = (oc[rows].double() - r["o"]).abs().max().item()
    el = (lc[:, rows].double() - r["lse"]).abs().max().item()
    dqg = dq.float().cpu()[rows].double()
    edq = ((dqg - r["dq"]).abs() - ULP[dtype] * r["dq"].abs()).max().item()
    print(f"  sampled rows: max|dO|={eo:.3e} max|dLSE|={el:.3e} dQ excess={edq:.3e}", flush=True)
    assert eo <= TOL[dtype] and el <= 1e-3 and edq <= TOL[dtype]

    # block 0: every query selects it (N * g rows, many work-groups, fp32 partials + reduce kernel)
    nblk = (n + bk - 1) // bk
    worst = {"dk": 0.0, "dv": 0.0}
    for kh in sorted({0, hkv - 1}):
        users = sel_tokens[kh][: int(counts[kh, 0])]
        assert len(users) == n
        dk0, dv0 = orc.key_block_grads_ref(q, k, v, do, oc, lc, kh, 0, users, bk, n, round_dtype=dtype)
        for nm, got, want in (("dk", dk, dk0), ("dv", dv, dv0)):
            gb = got[:bk, kh].float().cpu().double()
            err = (gb - want).abs().max().item()
            ex = ((gb - want).abs() - ULP[dtype] * want.abs()).max().item()
            worst[nm] = max(worst[nm], err)
            print(f"  block 0 kv head {kh} ({n} queries): {nm} max err {err:.3e} (|ref| max {want.abs().max().item():.1f})", flush=True)
            assert ex <= TOL[dtype], (nm, 0, ex)

    # moderately shared key blocks through the per-row oracle
    for kh, blk in [(0, nblk // 8), (hkv - 1, nblk // 2), (0, nblk - 1)]:
        s0 = int(starts[kh, blk])
        users = sel_tokens[kh][s0 : s0 + int(counts[kh, blk])].tolist()
        rb = orc.selected_attention_rows_ref(q, k, v, topk, bk, cu, users, do=do, o_in=oc, lse_in=lc,
                                             round_dtype=dtype, key_block=(kh, blk * bk))
        for nm, got, want in (("dk", dk, rb["dk_block"]), ("dv", dv, rb["dv_block"])):
            gb = got[blk * bk : (blk + 1) * bk, kh].float().cpu().double()
            ex = ((gb - want).abs() - ULP[dtype] * want.abs()).max().item()
            worst[nm] = max(worst[nm], (gb - want).abs().max().item())
            print(f"  block {blk} kv head {kh} ({len(users)} queries): {nm} max err {(gb - want).abs().max().item():.3e}", flush=True)
            assert ex <= TOL[dtype], (nm, blk, ex)
    edq_abs = (dqg - r["dq"]).abs().max().item()
    print(f"MAXABS {name}: O {eo:.2e} LSE {el:.2e} dQ {edq_abs:.2e} dK {worst['dk']:.2e} dV {worst['dv']:.2e} "
          f"(sampled rows / blocks incl. block 0)", flush=True)


def test_decode_full_size(dev):
    """One decode step at the full serving shape: 64 requests, cache lengths uniform in [32768, 131072], Hq=32,
    Hkv=8, D=128, compression 32/16, B_K=64, T=16, bf16.  Caches are drawn on the device (21 GB); the oracle is run
    on sampled requests (shortest, longest, first, last) from their slices, the top-k rule on every request, and
    the batch is checked for independence of its requests (a sub-batch gives the same results up to rounding)."""
    from oracle import decode as dorc
    hq, hkv, d, bk, t, ks, st = 32, 8, 128, 64, 16, 32, 16
    nreq = 64
    gen = torch.Generator().manual_seed(31)
    lens = torch.randint(32768, 131073, (nreq,), generator=gen).tolist()
    cu_k, cu_ck = [0], [0]
    for l in lens:
        cu_k.append(cu_k[-1] + l)
        cu_ck.append(cu_ck[-1] + (l - ks) // st + 1)
    print(f"case decode B={nreq} total cache rows {cu_k[-1]} compressed rows {cu_ck[-1]}", flush=True)
    torch.manual_seed(32)
    q = torch.randn(nreq, hq, d, device=dev, dtype=torch.bfloat16)
    kc = torch.randn(cu_k[-1], hkv, d, device=dev, dtype=torch.bfloat16)
    vc = torch.randn(cu_k[-1], hkv, d, device=dev, dtype=torch.bfloat16)
    ck = torch.randn(cu_ck[-1], hkv, d, device=dev, dtype=torch.bfloat16)
    cv = torch.randn(cu_ck[-1], hkv, d, device=dev, dtype=torch.bfloat16)
    pos = torch.tensor([l - 1 for l in lens], dtype=torch.int32, device=dev)
    seqlens = torch.tensor(lens, dtype=torch.int32, device=dev)
    cu_k_t = torch.tensor(cu_k, dtype=torch.int32, device=dev)
    cu_ck_t = torch.tensor(cu_ck, dtype=torch.int32, device=dev)
    max_ck = max(b_ - a_ for a_, b_ in zip(cu_ck[:-1], cu_ck[1:]))
    nblk_max = max(math.ceil(l / bk) for l in lens)

    def step(sl):
        b0, b1 = sl.start, sl.stop
        cck = (cu_ck_t[b0 : b1 + 1] - cu_ck_t[b0]).contiguous()
        ckk = (cu_k_t[b0 : b1 + 1] - cu_k_t[b0]).contiguous()
        o_c, lse_c, raw = ops.decode_cmpattn(q[sl], ck[cu_ck[b0]:cu_ck[b1]], cv[cu_ck[b0]:cu_ck[b1]], cck, pos[sl],
                                             ks, st, max_ck)
        idx, bscore = ops.decode_topk(raw, lse_c, cck, pos[sl], seqlens[sl], hq, ks, st, bk, t, nblk_max,
                                      softmax_scale=1.0 / math.sqrt(d), return_block_score=True)
        o_s, lse_s = ops.decode_selattn(q[sl], kc[cu_k[b0]:cu_k[b1]], vc[cu_k[b0]:cu_k[b1]], ckk, idx, bk)
        return o_c, lse_c, idx, bscore, o_s, lse_s

    full = step(slice(0, nreq))
    part = step(slice(5, 13))
    torch.cuda.synchronize()
    # The key tiles of the whole batch are dealt to the resident waves in equal shares, so where the fp32 partials
    # of a request are cut depends on the batch: a sub-batch agrees to rounding (one ulp of the bf16 output, 1e-5 in
    # the LSE, one bf16 ulp in the block scores).
    o_cf, lse_cf, idx_f, bs_f, o_sf, lse_sf = (a[5:13] if a.shape[0] == nreq else a[:, 5:13] for a in full)
    o_cp, lse_cp, idx_p, bs_p, o_sp, lse_sp = part
    assert (o_cf.float() - o_cp.float()).abs().max().item() <= 2.0 ** -7 * o_cf.float().abs().max().item()
    assert (lse_cf - lse_cp).abs().max().item() <= 1e-5
    fin = torch.isfinite(bs_f)
    assert torch.equal(fin, torch.isfinite(bs_p))
    assert ((bs_f[fin] - bs_p[fin]).abs() <= 2.0 ** -7 * bs_f[fin].abs()).all()
    # the selection is the top-k rule applied to the block scores of its own run; between the two runs it may differ
    # only where scores one bf16 ulp apart change places
    assert torch.equal(idx_p.cpu(), dorc.decode_topk_ref(bs_p.cpu(), t))
    same_idx = (idx_f == idx_p).all(-1)                      # [Hkv, 8]
    print(f"  selection identical for {same_idx.float().mean().item():.0%} of the (kv head, request) pairs", flush=True)
    assert same_idx.float().mean().item() >= 0.75
    rows = same_idx.all(0)                                   # requests whose selection agrees for every kv head
    assert rows.any()
    assert (o_sf[rows].float() - o_sp[rows].float()).abs().max().item() <= 2.0 ** -7 * o_sf.float().abs().max().item()
    assert (lse_sf[:, rows] - lse_sp[:, rows]).abs().max().item() <= 1e-5
    o_c, lse_c, idx, bscore, o_s, lse_s = full
    assert torch.isfinite(o_c.float()).all() and torch.isfinite(o_s.float()).all()
    assert torch.equal(idx.cpu(), dorc.decode_topk_ref(bscore.cpu(), t))
    # every request keeps block 0 and its last two blocks (init_blocks = 1, local_blocks = 2)
    own = (seqlens.long() - 1) // bk
    for forced in (torch.zeros_like(own), own, own - 1):
        assert (idx.long() == forced[None, :, None]).any(-1).all()
    order = sorted(range(nreq), key=lambda i: lens[i])
    for b in sorted({order[0], order[-1], 0, nreq - 1}):
        qb = q[b : b + 1].float().cpu()
        ckb, cvb = (x[cu_ck[b]:cu_ck[b + 1]].float().cpu() for x in (ck, cv))
        n_ck = cu_ck[b + 1] - cu_ck[b]
        o_r, lse_r = dorc.decode_compressed_attention_ref(qb, ckb, cvb, [0, n_ck], [lens[b] - 1], ks, st)
        e1 = (o_c[b : b + 1].float().cpu() - o_r).abs().max().item()
        e2 = (lse_c[:, b : b + 1].cpu() - lse_r).abs().max().item()
        bs_r = dorc.decode_block_scores_ref(qb, ckb, lse_r, [0, n_ck], [lens[b] - 1], [lens[b]], ks, st, bk,
                                            nblk_cols=nblk_max)
        got = bscore[:, b : b + 1].cpu()
        assert torch.equal(torch.isinf(got), torch.isinf(bs_r))
        fin = torch.isfinite(bs_r)
        e3 = (got[fin] - bs_r[fin]).abs().max().item()
        kcb, vcb = (x[cu_k[b]:cu_k[b + 1]].cpu() for x in (kc, vc))
        o_sr, lse_sr = dorc.decode_selected_attention_ref(qb, kcb, vcb, [0, lens[b]], idx[:, b : b + 1].cpu(), bk)
        e4 = (o_s[b : b + 1].float().cpu() - o_sr).abs().max().item()
        e5 = (lse_s[:, b : b + 1].cpu() - lse_sr).abs().max().item()
        print(f"  request {b} (len {lens[b]}): cmp dO {e1:.2e} dLSE {e2:.2e} block-score {e3:.2e}; "
              f"sel dO {e4:.2e} dLSE {e5:.2e}", flush=True)
        assert e1 <= 2e-2 and e2 <= 1e-3 and e3 <= 2e-3 and e4 <= 2e-2 and e5 <= 1e-3


def test_module_full_size(dev):
    """The Llama-3-8B-like layer at its full shape (hidden 4096, 32 / 8 heads of 128, compression 32/16, B_K=64,
    T=16, window 512; 4 sequences of 8192 tokens, bf16), forward and backward.  Every branch is causal, so the
    output of the first 1024 tokens of a sequence depends on those tokens only: that prefix is checked against the
    CPU oracle of the layer, for the first and the last sequence; the varlen batch is checked against a run of one
    of its sequences alone."""
    from fsa.module.fsa import FlashSparseAttention, RopeConfig
    from oracle import module as morc
    torch.manual_seed(3)
    cfg = dict(hidden_size=4096, num_q_heads=32, num_kv_heads=8, head_dim=128, kernel_size=32, kernel_stride=16,
               block_size=64, topk=16, init_blocks=1, local_blocks=2, window_size=512)
    layer = FlashSparseAttention(**cfg, rope_config=RopeConfig(head_dim=128)).to(dev).to(torch.bfloat16)
    nseq, slen, pre = 4, 8192, 1024
    n = nseq * slen
    x = torch.randn(n, 4096, device=dev, dtype=torch.bfloat16, requires_grad=True)
    cu = torch.arange(0, n + 1, slen, dtype=torch.int32, device=dev)
    print(f"case module {nseq} x {slen}", flush=True)
    y, topk_idx = layer(x, cu, return_topk_idx=True)
    (y.float() * torch.randn_like(y, dtype=torch.float32)).sum(-1).mean().backward()
    torch.cuda.synchronize()
    assert torch.isfinite(y.float()).all() and torch.isfinite(x.grad.float()).all()
    for name, p in layer.named_parameters():
        assert p.grad is not None and torch.isfinite(p.grad.float()).all() and p.grad.abs().max() > 0, name

    def rel(a, b):
        return ((a.float() - b.float()).norm() / b.float().norm()).item()

    with torch.no_grad():
        y1 = layer(x[2 * slen : 3 * slen].detach(), cu[:2])
    e = rel(y[2 * slen : 3 * slen], y1)
    print(f"  sequence 2 alone vs in the batch: rel {e:.3e}", flush=True)
    assert e < 1e-2
    params = {k: v.detach().float().cpu() for k, v in layer.named_parameters()}
    ocfg = dict(cfg, inv_freq=morc.llama3_inv_freq(128, 500000.0))
    for s in (0, nseq - 1):
        xs = x[s * slen : s * slen + pre].detach().float().cpu()
        y_r, _, _ = morc.fsa_layer_ref(params, xs, [0, pre], ocfg, topk_idx=topk_idx[:, s * slen : s * slen + pre].cpu())
        e = rel(y[s * slen : s * slen + pre].cpu(), y_r)
        print(f"  sequence {s} first {pre} tokens vs oracle: rel {e:.3e}", flush=True)
        assert e < 2e-2
