#!/usr/bin/env python3
"""Benchmark of the selected-attention hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

One "step" = index build + forward + backward of NSA selected attention for the
three GQA groups of the headline configuration (single varlen sequence of 65536
tokens, 4 kv heads, Hq = 4 / 8 / 16, head_dim 128, block 64, top-16, bf16,
synthetic N(0,1) inputs and the seeded synthetic block lists).  Inputs are
resident in HBM before the timed region.  Prints ONE JSON line.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "flash-sparse-attention_amd"))

MFMA_PEAK_TFLOPS = 2500.0   # MI355X dense bf16/fp16
HBM_PEAK_GBS = 8000.0       # MI355X HBM3E

# HBM bytes per launch at the default workload from two rocprofv3 --pmc passes over this script
# (FETCH_SIZE, WRITE_SIZE; KiB per dispatch), each scaled by the factor that makes the same counter
# read 1 GiB for the 1 GiB device copy of --calib-copy (FETCH_SIZE x 2.0, WRITE_SIZE x 1.0).
PMC_TRAFFIC_BYTES = {
    ("selattn_bwd_dqdkdv", 4): 13549486080,
    ("selattn_bwd_dqdkdv", 2): 6610281472,
    ("selattn_bwd_dqdkdv", 1): 3254586368,
    ("selattn_fwd_main", 4): 8274831360,
    ("selattn_fwd_main", 2): 4033090560,
    ("selattn_fwd_main", 1): 1987578880,
    ("selattn_fwd_reduce", 4): 4978273280,
    ("selattn_bwd_dq_reduce", 4): 4650569728,
}

METRIC = "selected-attn fwd+bwd ms & TFLOP/s at 64K, B_K=64, T=16, GQA 1-4; roofline %"


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--seq-len", type=int, default=65536)
    ap.add_argument("--groups", type=str, default="1,2,4")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-seq-len", type=int, default=8192)
    ap.add_argument("--workload", choices=["c1", "c3", "module", "decode"], default="c1",
                    help="c1 = the headline configuration (default); the others time the remaining parity "
                         "configurations (large-head fp16 selected attention, the full layer, one decode step)")
    ap.add_argument("--calib-copy", action="store_true",
                    help="issue three 1 GiB device copies first (known-size reference for hardware counters)")
    return ap.parse_args()


def cpu_baseline(seq_len: int, d: int, bk: int, topk: int, hkv: int):
    """The CPU oracle (a PyTorch-eager port of the reference's math) timed on the host cores:
    forward + backward of the same operator on a bounded sample of the workload."""
    import torch
    from synth_inputs import make_qkv, make_topk_idx
    from oracle import selattn as orc

    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    cu = [0, seq_len]
    q, k, v, do = make_qkv(seq_len, hkv, hkv, d, torch.float32, seed=0)
    idx = make_topk_idx(cu, hkv, bk, topk, seed=1)
    _, p_key = orc.count_pairs(idx, bk, cu)
    flops = 14.0 * d * p_key  # summed over heads already (g = 1)
    times = []
    for _ in range(2):
        t0 = time.perf_counter()
        orc.selected_attention_grads_ref(q, k, v, idx, bk, cu, do)
        times.append(time.perf_counter() - t0)
    best = min(times)
    return {
        "value": flops / best / 1e12,
        "unit": "TFLOP/s",
        "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": f"oracle fwd+bwd (fp32 eager PyTorch), 1 sequence S={seq_len}, Hkv=Hq={hkv}, D={d}, "
                  f"B_K={bk}, T={topk}; best of 2 runs, {best * 1e3:.0f} ms",
        "ms": best * 1e3,
    }


def _kernel_records(kern, algo):
    """[{kernel, ms, bound, achieved, peak, unit, frac, algo_tflops, algo_gbs}] sorted by time; `algo` maps a
    label to (flops, bytes) of one step, or None where no closed form is given (GEMMs of the library etc.)."""
    out = []
    for name, ms in sorted(kern.items(), key=lambda kv: -kv[1]):
        rec = {"kernel": name, "ms": round(ms, 4)}
        ab = algo.get(name)
        if ab is not None and ms > 0:
            fl, by = ab
            tf, gbs = fl / (ms * 1e-3) / 1e12, by / (ms * 1e-3) / 1e9
            if tf / MFMA_PEAK_TFLOPS > gbs / HBM_PEAK_GBS:
                rec.update(bound="mfma", achieved=round(tf, 2), peak=MFMA_PEAK_TFLOPS, unit="TFLOP/s",
                           frac=round(tf / MFMA_PEAK_TFLOPS, 4))
            else:
                rec.update(bound="hbm", achieved=round(gbs, 2), peak=HBM_PEAK_GBS, unit="GB/s",
                           frac=round(gbs / HBM_PEAK_GBS, 4))
            rec.update(algo_tflops=round(tf, 2), algo_gbs=round(gbs, 1))
        out.append(rec)
    return out


def side_workload(args):
    """Timing of the two parity configurations that are not selected attention alone: the full layer
    (forward + backward, 4 x 8192 tokens) and one decode step (64 requests).  Same JSON shape, value in ms;
    every library kernel is listed with its duration and, where its least work has a closed form, with the
    roofline it sits closer to (algorithmic flops against the MFMA peak, algorithmic bytes against HBM)."""
    import math
    import torch
    from fsa_hip import _lib, ops
    dev = torch.device("cuda:0")
    torch.manual_seed(0)
    e = 2
    algo = {}
    if args.workload == "module":
        from fsa.module.fsa import FlashSparseAttention, RopeConfig
        hidden, hq, hkv, d, ks, st, bk, t, win, nseq, slen = 4096, 32, 8, 128, 32, 16, 64, 16, 512, 4, 8192
        layer = FlashSparseAttention(hidden_size=hidden, num_q_heads=hq, num_kv_heads=hkv, head_dim=d, kernel_size=ks,
                                     kernel_stride=st, block_size=bk, topk=t, init_blocks=1, local_blocks=2,
                                     window_size=win, rope_config=RopeConfig(head_dim=d)).to(dev).to(torch.bfloat16)
        n = nseq * slen
        x = torch.randn(n, hidden, device=dev, dtype=torch.bfloat16, requires_grad=True)
        w = torch.randn(n, hidden, device=dev, dtype=torch.bfloat16)
        cu = torch.arange(0, n + 1, slen, dtype=torch.int32, device=dev)
        name = "FlashSparseAttention layer fwd+bwd, hidden 4096, Hq=32, Hkv=8, D=128, 32/16 compression, B_K=64, " \
               "T=16, window 512, 4 x 8192 tokens"

        def step():
            layer.zero_grad(set_to_none=True)
            x.grad = None
            (layer(x, cu) * w).sum().backward()

        # least work per kernel label (one step; a label covers every launch of that kernel in the step)
        g = hq // hkv
        nc = (slen - ks) // st + 1
        i = torch.arange(slen)
        vis_c = int(torch.clamp((i - ks + 1) // st + 1, 0, nc).sum()) * nseq        # (query, compressed key) pairs
        vis_w = int((torch.clamp(i, max=win) + 1).sum()) * nseq                     # (query, key) pairs of the band
        with torch.no_grad():
            _, idx = layer(x, cu, return_topk_idx=True)
        idx = idx.cpu()
        ok = idx >= 0
        pos = torch.arange(slen).repeat(nseq)[None, :, None]
        lo = idx.long() * bk
        nkeys = (torch.minimum(pos, lo + bk - 1) - lo + 1).clamp(min=0)
        pairs = int(ok.sum())                                                        # summed over kv heads
        p_key = int(torch.where(ok, nkeys, torch.zeros_like(nkeys)).sum())
        rows = pairs * g
        qbytes = n * hq * d * e
        kvbytes = 2 * n * hkv * d * e
        ckv = 2 * nseq * nc * hkv * d * e
        algo.update({
            "selattn_fwd_main": (4.0 * d * p_key * g, rows * (2 * d * e + 4) + kvbytes),
            "selattn_fwd_reduce": (0.0, rows * (d * e + 4) + n * hq * (d * e + 4)),
            "selattn_bwd_dqdkdv": (10.0 * d * p_key * g, rows * (3 * d * e + 8) + 2 * kvbytes),
            "selattn_bwd_dq_reduce": (0.0, rows * d * e + qbytes),
            "selattn_bwd_delta": (0.0, 2 * qbytes + 4 * n * hq),
            "cmpattn_bwd_delta": (0.0, 2 * qbytes + 4 * n * hq),
            "winattn_bwd_delta": (0.0, 2 * qbytes + 4 * n * hq),
            "cmpattn_fwd": (4.0 * d * vis_c * hq, 2 * qbytes + ckv),
            "cmpattn_bwd_dq": (6.0 * d * vis_c * hq, 3 * qbytes + ckv),
            "cmpattn_bwd_dkdv": (8.0 * d * vis_c * hq, 2 * qbytes + 2 * ckv),
            "winattn_fwd": (4.0 * d * vis_w * hq, 2 * qbytes + kvbytes),
            "winattn_bwd_dq": (6.0 * d * vis_w * hq, 3 * qbytes + kvbytes),
            "winattn_bwd_dkdv": (8.0 * d * vis_w * hq, 2 * qbytes + 2 * kvbytes),
            "cmp_score": (2.0 * d * vis_c * hkv, n * hkv * d * e + 4.0 * hkv * n * (nc // 4 + 1)),  # q in, fp32 block scores out
            "cmp_topk": (0.0, 4.0 * hkv * n * (nc // 4 + 1) + 4.0 * hkv * n * t),    # ... read back, ids written
            "rope": (0.0, 2.0 * (2 * qbytes + 2 * n * hkv * d * e + 2 * nseq * nc * hkv * d * e)),  # fwd + bwd, in + out
            "gate_merge_fwd": (0.0, 4.0 * qbytes),
            "gate_merge_bwd": (0.0, 7.0 * qbytes),
            "linear_compress_fwd": (2 * 2.0 * nseq * nc * ks * d * d * hkv, kvbytes + ckv + 2 * hkv * ks * d * d * e),
            "linear_compress_dx": (2 * 2.0 * nseq * nc * ks * d * d * hkv, kvbytes + ckv + 2 * hkv * ks * d * d * e),
            "linear_compress_dw": (2 * 2.0 * nseq * nc * ks * d * d * hkv, kvbytes + ckv + 2 * hkv * ks * d * d * 4),
            "index_build": (0.0, 4.0 * hkv * n * t * 2 + 4.0 * pairs),
        })
    else:
        hq, hkv, d, bk, t, ks, st, nreq = 32, 8, 128, 64, 16, 32, 16, 64
        gen = torch.Generator().manual_seed(31)
        lens = torch.randint(32768, 131073, (nreq,), generator=gen).tolist()
        cu_k, cu_ck = [0], [0]
        for l in lens:
            cu_k.append(cu_k[-1] + l)
            cu_ck.append(cu_ck[-1] + (l - ks) // st + 1)
        q = torch.randn(nreq, hq, d, device=dev, dtype=torch.bfloat16)
        kc, vc = (torch.randn(cu_k[-1], hkv, d, device=dev, dtype=torch.bfloat16) for _ in range(2))
        ck, cv = (torch.randn(cu_ck[-1], hkv, d, device=dev, dtype=torch.bfloat16) for _ in range(2))
        pos = torch.tensor([l - 1 for l in lens], dtype=torch.int32, device=dev)
        seqlens = torch.tensor(lens, dtype=torch.int32, device=dev)
        cu_k_t = torch.tensor(cu_k, dtype=torch.int32, device=dev)
        cu_ck_t = torch.tensor(cu_ck, dtype=torch.int32, device=dev)
        max_ck = max(b - a for a, b in zip(cu_ck[:-1], cu_ck[1:]))
        nblk_max = max(math.ceil(l / bk) for l in lens)
        name = f"one decode step (compressed attention, top-k, selected attention), {nreq} requests, caches " \
               f"32768-131072 ({cu_k[-1]} rows), Hq=32, Hkv=8, D=128, B_K=64, T=16"

        def step():
            o_c, lse_c, raw = ops.decode_cmpattn(q, ck, cv, cu_ck_t, pos, ks, st, max_ck)
            idx = ops.decode_topk(raw, lse_c, cu_ck_t, pos, seqlens, hq, ks, st, bk, t, nblk_max,
                                  softmax_scale=1.0 / math.sqrt(d))
            ops.decode_selattn(q, kc, vc, cu_k_t, idx, bk)

        n_vis = sum(min((l - ks) // st + 1, (l - 1 - ks + 1) // st + 1) for l in lens)   # visible compressed keys
        algo.update({
            "decode_cmpattn": (4.0 * d * n_vis * hq, 2.0 * n_vis * hkv * d * e),       # K and V rows, once
            "decode_selattn": (4.0 * d * nreq * t * bk * hq, 2.0 * nreq * t * bk * hkv * d * e),
            "decode_topk": (0.0, 4.0 * hkv * n_vis),
        })
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / args.steps
    _lib.profile_enable(True)
    step()
    torch.cuda.synchronize()
    recs = _lib.profile_records()
    _lib.profile_enable(False)
    kern = {}
    for nm, t_ in recs:
        kern[nm] = kern.get(nm, 0.0) + t_
    kernels = _kernel_records(kern, algo)
    lib_ms = sum(kern.values())
    print(json.dumps({"metric": "ms per step", "value": round(ms, 4), "unit": "ms", "n_gpus": 1, "steps": args.steps,
                      "warmup": args.warmup, "ms_per_step": round(ms, 4), "higher_is_better": False,
                      "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
                      "config": {"workload": name},
                      "library_kernels_ms_total": round(lib_ms, 4),
                      "other_ms": round(ms - lib_ms, 4),   # projections on the BLAS library, autograd glue
                      "kernels": kernels}))


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (every box has one GPU); run with --gpus 1",
              file=sys.stderr)
        sys.exit(2)
    if args.workload in ("module", "decode"):
        return side_workload(args)
    import torch
    from fsa.ops.FSA_topk_sparse_attention import (_topk_sparse_attention_bwd_opt,
                                                   _topk_sparse_attention_fwd_opt)
    from fsa_hip import _lib, ops
    from synth_inputs import make_qkv, make_topk_idx

    assert torch.cuda.is_available(), "bench.py needs a ROCm device"
    dev = torch.device("cuda:0")
    n, hkv, d, bk, topk = args.seq_len, 4, 128, 64, 16
    groups = [int(x) for x in args.groups.split(",")]
    dtype, std = torch.bfloat16, 1.0
    if args.workload == "c3":           # large heads: fp16, D=256, Hkv=2, GQA 2, S=131072, B_K=128, T=8, sigma 0.5
        n, hkv, d, bk, topk, groups, dtype, std = 131072, 2, 256, 128, 8, [2], torch.float16, 0.5
    scale = 1.0 / d ** 0.5
    cu = [0, n]
    cu_t = torch.tensor(cu, dtype=torch.int32, device=dev)
    idx_cpu = make_topk_idx(cu, hkv, bk, topk, seed=1)
    idx = idx_cpu.to(dev)
    # exact work: valid (query, block) pairs and unmasked (query, key) pairs, summed over kv heads
    own = torch.arange(n) // bk
    lo = idx_cpu.long() * bk
    ok = idx_cpu >= 0
    nkeys = (torch.minimum(torch.arange(n)[None, :, None], lo + bk - 1) - lo + 1).clamp(min=0)
    pairs = int(ok.sum())
    p_key = int(torch.where(ok, nkeys, torch.zeros_like(nkeys)).sum())
    nblk = (n + bk - 1) // bk
    del own, lo, ok, nkeys

    if args.calib_copy:
        a = torch.ones(1 << 28, dtype=torch.float32, device=dev)
        b = torch.empty_like(a)
        for _ in range(3):
            b.copy_(a)
        torch.cuda.synchronize()
        del a, b

    data = {}
    for g in groups:
        data[g] = tuple(x.to(dev) for x in make_qkv(n, hkv * g, hkv, d, dtype, seed=100 + g, std=std))

    def run_g(g):
        q, k, v, do = data[g]
        o, lse, perm = _topk_sparse_attention_fwd_opt(q, k, v, idx, bk, cu_t, cu_t, n, n, scale)
        return _topk_sparse_attention_bwd_opt(o, do, lse, q, k, v, idx, bk, cu_t, cu_t, n, n, scale, perm)

    def step():
        for g in groups:
            run_g(g)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps

    flops_g = {g: 14.0 * d * p_key * g for g in groups}
    total_tflop = sum(flops_g.values()) / 1e12
    value = total_tflop / (ms_per_step * 1e-3)

    # per-kernel durations from HIP events recorded on the launch stream inside the library
    _lib.profile_enable(True)
    reps = max(3, min(10, args.steps))
    for _ in range(reps):
        for g in groups:
            run_g(g)
    torch.cuda.synchronize()
    recs = _lib.profile_records()
    _lib.profile_enable(False)
    per_call = len(recs) // (reps * len(groups))
    kern = {}
    for i, (name, ms) in enumerate(recs):
        g = groups[(i // per_call) % len(groups)]
        kern.setdefault((name, g), []).append(ms)
    kern = {k_: sum(v_) / len(v_) for k_, v_ in kern.items()}

    e = 2  # bytes per element
    kv_once = 2 * n * hkv * d * e          # K and V (or dK and dV) of every kv head, once

    def algo(name, g):
        """(flops, bytes) one launch must do at the least: MFMA flops over unmasked (query, key) pairs,
        HBM bytes of the tensors it has to read and write once."""
        hq = hkv * g
        pg = pairs * g                      # (query, head, block) rows
        if name == "selattn_fwd_main":      # S = QK^T, O = PV; Q row in, normalised partial row + lse out
            return 4.0 * d * p_key * g, pg * (2 * d * e + 4) + kv_once
        if name == "selattn_bwd_dqdkdv":    # S, dP, dV, dK, dQ; Q, dO rows in, dQ partial row out, lse + delta in
            return 10.0 * d * p_key * g, pg * (3 * d * e + 8) + 2 * kv_once
        if name == "selattn_bwd_dq":
            return 6.0 * d * p_key * g, pg * (3 * d * e + 8) + kv_once
        if name == "selattn_bwd_dkdv":
            return 8.0 * d * p_key * g, pg * (2 * d * e + 8) + 2 * kv_once
        if name == "selattn_fwd_reduce":
            return 0.0, pg * (d * e + 4) + n * hq * (d * e + 4)
        if name == "selattn_bwd_dq_reduce":
            return 0.0, pg * d * e + n * hq * d * e
        if name == "selattn_bwd_delta":
            return 0.0, 2 * n * hq * d * e + n * hq * 4
        if name == "index_build":
            return 0.0, 4 * hkv * n * topk * 2 + 4 * (pairs + 2 * nblk * hkv)
        # selattn_bwd_dkdv_reduce: no least work of its own - dK / dV written once are counted in the fused
        # kernel; it only adds up the fp32 partials of blocks that were split over several work-groups
        return 0.0, 0.0

    kernels = []
    for (name, g), ms in sorted(kern.items(), key=lambda kv: -kv[1]):
        fl, by = algo(name, g)
        tf, gbs = fl / (ms * 1e-3) / 1e12, by / (ms * 1e-3) / 1e9
        f_mfma, f_hbm = tf / MFMA_PEAK_TFLOPS, gbs / HBM_PEAK_GBS
        rec = {"kernel": name, "gqa": g, "ms": round(ms, 4)}
        if fl == 0 and by == 0:
            kernels.append(rec)
            continue
        if f_mfma > f_hbm:                  # the roofline that binds is the one the kernel sits closer to
            rec.update(bound="mfma", achieved=round(tf, 2), peak=MFMA_PEAK_TFLOPS, unit="TFLOP/s", frac=round(f_mfma, 4))
        else:
            rec.update(bound="hbm", achieved=round(gbs, 2), peak=HBM_PEAK_GBS, unit="GB/s", frac=round(f_hbm, 4))
        rec.update(algo_tflops=round(tf, 2), algo_gbs=round(gbs, 1), algo_bytes=int(by))
        kernels.append(rec)
    dom = kernels[0]
    traffic = PMC_TRAFFIC_BYTES.get((dom["kernel"], dom["gqa"])) if (n, d, bk, topk) == (65536, 128, 64, 16) else None
    roofline = {"kernel": f"{dom['kernel']} (GQA {dom['gqa']})", "bound": dom["bound"],
                "achieved": dom["achieved"], "peak": dom["peak"], "unit": dom["unit"], "frac": dom["frac"],
                "traffic": traffic}

    per_gqa = []
    for g in groups:
        parts = {nm: ms for (nm, gg), ms in kern.items() if gg == g}
        fwd = parts.get("selattn_fwd_main", 0) + parts.get("selattn_fwd_reduce", 0)
        bwd = sum(ms for nm, ms in parts.items() if nm.startswith("selattn_bwd"))
        tot = fwd + bwd + parts.get("index_build", 0)
        per_gqa.append({"gqa": g, "hq": hkv * g, "index_ms": round(parts.get("index_build", 0), 4),
                        "fwd_ms": round(fwd, 4), "bwd_ms": round(bwd, 4),
                        "tflops": round(flops_g[g] / 1e12 / (tot * 1e-3), 2),
                        "mfma_frac": round(flops_g[g] / 1e12 / (tot * 1e-3) / MFMA_PEAK_TFLOPS, 4)})

    out = {
        "metric": METRIC,
        "value": round(value, 2),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16" if dtype == torch.bfloat16 else "fp16",
        "data": "synthetic",
        "config": {"workload": f"selected attention index+fwd+bwd, 1 varlen sequence S={n}, Hkv={hkv}, "
                               f"GQA {'/'.join(map(str, groups))} swept in one step, D={d}, B_K={bk}, T={topk}",
                   "pairs_per_kv_head": pairs // hkv, "unmasked_qk_pairs_per_q_head": p_key // hkv,
                   "tflop_per_step": round(total_tflop, 4), "seed": 1},
        "mfma_frac_whole_step": round(value / MFMA_PEAK_TFLOPS, 4),
        "roofline": roofline,
        "per_gqa": per_gqa,
        "kernels": kernels,
    }
    if not args.no_cpu_baseline and args.workload == "c1":
        out["cpu_baseline"] = cpu_baseline(args.cpu_seq_len, d, bk, topk, hkv)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
