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

# Kernels whose least work is a dense 16-bit contraction are priced against the MFMA peak (with the HBM view
# beside it), the streaming / gathering / integer kernels against the HBM peak.
MFMA_KERNELS = {"selattn_fwd_main", "selattn_bwd_dqdkdv", "cmpattn_fwd", "cmpattn_bwd_dq", "cmpattn_bwd_dkdv",
                "winattn_fwd", "winattn_bwd_dq", "winattn_bwd_dkdv", "cmp_score", "linear_compress_fwd",
                "linear_compress_dx", "linear_compress_dw"}

# Measured HBM traffic per launch comes from the committed counter summary of this same script (two rocprofv3
# --pmc passes, FETCH_SIZE and WRITE_SIZE, scaled by what the counters read for a 1 GiB device copy); the file
# is read at run time, so a kernel without a line there reports null instead of a stale figure.
TRAFFIC_FILES = {"c1": "selattn_fwd_bwd_S65536_bf16_hbm_traffic_pmc.txt"}
TRAFFIC_KERNEL_NAMES = {"selattn_bwd_dqdkdv": "attn_bwd_dkdv_kernel", "selattn_fwd_main": "selattn_fwd_main_kernel",
                        "selattn_fwd_reduce": "selattn_fwd_reduce_kernel",
                        "selattn_bwd_dq_reduce": "selattn_bwd_reduce_kernel",
                        "selattn_bwd_delta": "selattn_bwd_delta_kernel"}


# the sources that define the kernels of the selected-attention step (index, forward, backward)
SELATTN_SOURCES = ("fsa_common.h", "index.hip", "selattn_fwd.hip", "selattn_bwd.hip", "dkdv_kernel.h")


def csrc_sha16(names=SELATTN_SOURCES) -> str:
    """Hash of kernel sources under csrc/ (default: those of the selected-attention step; None: every .hip / .h):
    identifies the code a counter summary was captured from."""
    import hashlib
    h = hashlib.sha256()
    csrc = os.path.join(ROOT, "flash-sparse-attention_amd", "csrc")
    if names is None:
        names = sorted(f for f in os.listdir(csrc) if f.endswith((".hip", ".h")))
    for f in names:
        h.update(f.encode())
        h.update(open(os.path.join(csrc, f), "rb").read())
    return h.hexdigest()[:16]


def measured_traffic(workload: str):
    """({(label, gqa): bytes per launch}, source) from profiles/<summary>: lines `<kernel> grid=<n> gqa=<g> ...
    bytes=<x> GB`.  The summary names the kernel sources it was captured from (`# csrc_sha16: <hash>` over
    SELATTN_SOURCES); when those sources differ in this tree, nothing is returned - a stale figure is worse than
    none."""
    import re
    out = {}
    name = TRAFFIC_FILES.get(workload, "-")
    path = os.path.join(ROOT, "profiles", name)
    if not os.path.exists(path):
        return out, None
    text = open(path).read()
    m = re.search(r"^# csrc_sha16: (\w+)", text, re.M)
    sha, now = (m.group(1) if m else None), csrc_sha16()
    source = {"file": "profiles/" + name, "captured_from_csrc_sha16": sha, "this_tree_csrc_sha16": now,
              "how": "two rocprofv3 --pmc passes (FETCH_SIZE, WRITE_SIZE) over this script, read from the committed "
                     "summary - not measured in this run"}
    if sha != now:
        source["stale"] = True
        return out, source
    for line in text.splitlines():
        m = re.match(r"^(\S+)\s+grid=\s*\d+\s+gqa=(\d+)\s.*bytes=([0-9.]+) GB", line)
        if not m:
            continue
        for label, frag in TRAFFIC_KERNEL_NAMES.items():
            if frag in m.group(1):
                out[(label, int(m.group(2)))] = int(float(m.group(3)) * 1e9)
    return out, source

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


def cpu_baseline(d: int, bk: int, topk: int, hkv: int, c1_seq_len: int, c1_p_key_per_head: int, sample_seq_len: int):
    """The CPU oracle (a PyTorch-eager port of the reference's math; the reference has no CPU path of its own)
    timed on the host cores.  `value`: the CPU-plumbing configuration exactly - forward of one sequence S=4096,
    Hkv=Hq=4, fp32, median of 3.  Beside it the headline workload by extrapolation: forward + backward at
    S=sample_seq_len timed once, scaled linearly in the number of unmasked (query, key) pairs to S=c1_seq_len at
    GQA 1 (the cost of selected attention is linear in those pairs); labelled as an extrapolation."""
    import statistics
    import torch
    from synth_inputs import make_qkv, make_topk_idx
    from oracle import selattn as orc

    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    s0 = 4096
    q, k, v = make_qkv(s0, hkv, hkv, d, torch.float32, seed=0, with_do=False)
    idx = make_topk_idx([0, s0], hkv, bk, topk, seed=1)
    _, p_key0 = orc.count_pairs(idx, bk, [0, s0])
    times = []
    for _ in range(3):
        t0 = time.perf_counter()
        orc.selected_attention_ref(q, k, v, idx, bk, [0, s0])
        times.append(time.perf_counter() - t0)
    c0 = statistics.median(times)
    out = {
        "value": round(4.0 * d * p_key0 / c0 / 1e12, 5),
        "unit": "TFLOP/s",
        "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": f"oracle forward (fp32 eager PyTorch), 1 sequence S={s0}, Hkv=Hq={hkv}, D={d}, B_K={bk}, "
                  f"T={topk}: median of 3 runs {c0 * 1e3:.0f} ms",
        "ms": round(c0 * 1e3, 1),
    }
    s1 = sample_seq_len
    q, k, v, do = make_qkv(s1, hkv, hkv, d, torch.float32, seed=0)
    idx = make_topk_idx([0, s1], hkv, bk, topk, seed=1)
    _, p_key1 = orc.count_pairs(idx, bk, [0, s1])
    t0 = time.perf_counter()
    orc.selected_attention_grads_ref(q, k, v, idx, bk, [0, s1], do)
    t1 = time.perf_counter() - t0
    factor = c1_p_key_per_head * hkv / p_key1
    out["headline_extrapolated"] = {
        "note": f"EXTRAPOLATION: oracle forward+backward timed at S={s1} (GQA 1, {t1 * 1e3:.0f} ms, "
                f"{14.0 * d * p_key1 / t1 / 1e12:.4f} TFLOP/s), scaled by the ratio of unmasked (query, key) pairs "
                f"({factor:.2f}) to S={c1_seq_len} at GQA 1",
        "sample_ms": round(t1 * 1e3, 1),
        "gqa1_fwd_bwd_ms": round(t1 * factor * 1e3, 0),
    }
    return out


def parity_sample(run_g, data, g, idx_cpu, bk, n, dtype):
    """Plain max-abs differences of the device results of one GQA group of the timed workload against the CPU
    oracle: O / LSE / dQ on 32 seeded queries, dK / dV on key block 0 of kv head 0 (selected by every query: the
    block with the largest gradients) and on one block in the middle of the sequence.  Part of the CPU-baseline
    leg: the oracle is the checker here, nothing of it is timed as the product."""
    import torch
    from oracle import selattn as orc
    q, k, v, do = (x.cpu() for x in data[g])
    dq, dk, dv, o, lse = run_g(g, want_fwd=True)
    torch.cuda.synchronize()
    oc, lc = o.float().cpu(), lse.cpu()
    gen = torch.Generator().manual_seed(7)
    rows = sorted(set([0, bk, n - 1] + torch.randint(0, n, (29,), generator=gen).tolist()))
    cu = [0, n]
    r = orc.selected_attention_rows_ref(q, k, v, idx_cpu, bk, cu, rows, do=do, o_in=oc, lse_in=lc, round_dtype=dtype)
    out = {"gqa": g, "queries": len(rows),
           "max_abs_o": float((oc[rows].double() - r["o"]).abs().max()),
           "max_abs_lse": float((lc[:, rows].double() - r["lse"]).abs().max()),
           "max_abs_dq": float((dq.float().cpu()[rows].double() - r["dq"]).abs().max())}
    nblk = (n + bk - 1) // bk
    for blk in (0, nblk // 2):
        users = (idx_cpu[0] == blk).any(-1).nonzero().flatten()
        dk0, dv0 = orc.key_block_grads_ref(q, k, v, do, oc, lc, 0, blk * bk, users, bk, n, round_dtype=dtype)
        gk = dk[blk * bk:(blk + 1) * bk, 0].float().cpu().double()
        gv = dv[blk * bk:(blk + 1) * bk, 0].float().cpu().double()
        out[f"block{blk}"] = {"queries": int(users.numel()), "max_abs_dk": float((gk - dk0).abs().max()),
                              "max_abs_dv": float((gv - dv0).abs().max()),
                              "max_ref_dk": float(dk0.abs().max()), "max_ref_dv": float(dv0.abs().max())}
    out["note"] = ("plain max-abs, no ulp allowance; one bf16 ulp at |ref| = 8 is 0.0625, so the rounding of the "
                   "output alone can reach 0.031 there")
    return out


def _roofline_fields(name, ms, flops, nbytes):
    """Roofline entry of one kernel: against the MFMA peak for the contraction kernels, against HBM otherwise."""
    tf, gbs = flops / (ms * 1e-3) / 1e12, nbytes / (ms * 1e-3) / 1e9
    if name in MFMA_KERNELS:
        rec = dict(bound="mfma", achieved=round(tf, 2), peak=MFMA_PEAK_TFLOPS, unit="TFLOP/s",
                   frac=round(tf / MFMA_PEAK_TFLOPS, 4))
    else:
        rec = dict(bound="hbm", achieved=round(gbs, 2), peak=HBM_PEAK_GBS, unit="GB/s",
                   frac=round(gbs / HBM_PEAK_GBS, 4))
    rec.update(algo_tflops=round(tf, 2), algo_gbs=round(gbs, 1), algo_bytes=int(nbytes))
    return rec


def _kernel_records(kern, algo):
    """[{kernel, ms, bound, achieved, peak, unit, frac, algo_tflops, algo_gbs}] sorted by time; `algo` maps a
    label to (flops, bytes) of one step, or None where no closed form is given (GEMMs of the library etc.)."""
    out = []
    for name, ms in sorted(kern.items(), key=lambda kv: -kv[1]):
        rec = {"kernel": name, "ms": round(ms, 4)}
        ab = algo.get(name)
        if ab is not None and ms > 0:
            rec.update(_roofline_fields(name, ms, ab[0], ab[1]))
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
            "selattn_bwd_delta": (0.0, 2 * qbytes + 12 * n * hq),   # o, dO, lse in; (lse, delta) pairs out
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
    extra = {}
    if args.workload == "decode":
        # the same step recorded into a HIP graph (the lengths are device arrays, so a recorded step stays valid
        # while the caches grow): what the launches cost when they are issued one by one
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            step()
        for _ in range(args.warmup):
            graph.replay()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            graph.replay()
        torch.cuda.synchronize()
        extra["graph_replay_ms_per_step"] = round((time.perf_counter() - t0) * 1e3 / args.steps, 4)
    print(json.dumps({"metric": "ms per step", "value": round(ms, 4), "unit": "ms", "n_gpus": 1, "steps": args.steps,
                      "warmup": args.warmup, "ms_per_step": round(ms, 4), "higher_is_better": False,
                      "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
                      "config": {"workload": name},
                      "library_kernels_ms_total": round(lib_ms, 4),
                      "other_ms": round(ms - lib_ms, 4),   # projections on the BLAS library, autograd glue
                      **extra, "kernels": kernels}))


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

    def run_g(g, want_fwd=False):
        q, k, v, do = data[g]
        o, lse, perm = _topk_sparse_attention_fwd_opt(q, k, v, idx, bk, cu_t, cu_t, n, n, scale)
        grads = _topk_sparse_attention_bwd_opt(o, do, lse, q, k, v, idx, bk, cu_t, cu_t, n, n, scale, perm)
        return (*grads, o, lse) if want_fwd else grads

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

    # peak device memory of one group's index + forward + backward (inputs, outputs, index, partial buffers), as
    # the reference's harness prints it (test/test_FSA_module.py:137)
    peak_mem = {}
    for g in groups:
        torch.cuda.synchronize()
        torch.cuda.reset_peak_memory_stats()
        base = torch.cuda.memory_allocated()
        r_ = run_g(g)
        torch.cuda.synchronize()
        peak_mem[g] = {"max_memory_allocated": int(torch.cuda.max_memory_allocated()),
                       "above_resident_inputs": int(torch.cuda.max_memory_allocated() - base)}
        del r_

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
        """(flops, least bytes, gather-model bytes) of one launch.  flops: MFMA work over the unmasked (query, key)
        pairs.  least bytes: every input and output tensor once, plus the partial rows that the two-stage design
        writes in one kernel and reads in the next, plus the index lists.  gather-model bytes: the same with q / dO
        rows counted once per (query, block) pair, i.e. what the block-major kernels request when no gathered row
        is found in a cache - the distance between the two is the re-gather of query rows."""
        hq = hkv * g
        pg = pairs * g                      # (query, head, block) rows
        q_once = n * hq * d * e
        idx_lists = 4 * pairs + 8 * nblk * hkv
        if name == "selattn_fwd_main":      # S = QK^T, O = PV; q in, normalised partial row + lse out
            least = q_once + kv_once + pg * (d * e + 4) + idx_lists
            return 4.0 * d * p_key * g, least, least - q_once + pg * d * e
        if name == "selattn_bwd_dqdkdv":    # S, dP, dV, dK, dQ; q, dO, lse, delta, k, v in; dQ partial rows, dk, dv out
            least = 2 * q_once + 8 * n * hq + 2 * kv_once + pg * d * e + idx_lists
            return 10.0 * d * p_key * g, least, least - 2 * q_once - 8 * n * hq + pg * (2 * d * e + 8)
        if name == "selattn_fwd_reduce":
            by = pg * (d * e + 4) + n * hq * (d * e + 4) + 4 * hkv * n * topk
            return 0.0, by, by
        if name == "selattn_bwd_dq_reduce":
            by = pg * d * e + q_once + 4 * hkv * n * topk
            return 0.0, by, by
        if name == "selattn_bwd_delta":
            by = 2 * q_once + n * hq * 12    # o, dO, lse in; (lse, delta) pairs out
            return 0.0, by, by
        if name == "index_build":
            by = 4 * hkv * n * topk * 2 + 4 * (pairs + 2 * nblk * hkv)
            return 0.0, by, by
        return 0.0, 0.0, 0.0

    traffic_of, traffic_source = (measured_traffic(args.workload) if (n, d, bk, topk) == (65536, 128, 64, 16)
                                  else ({}, None))
    kernels = []
    for (name, g), ms in sorted(kern.items(), key=lambda kv: -kv[1]):
        fl, by, by_gather = algo(name, g)
        rec = {"kernel": name, "gqa": g, "ms": round(ms, 4)}
        if fl == 0 and by == 0:
            kernels.append(rec)
            continue
        rec.update(_roofline_fields(name, ms, fl, by))
        if name in MFMA_KERNELS:            # the HBM view beside the MFMA fraction, with both byte counts
            rec["hbm"] = {"least_bytes": int(by), "frac_least": round(by / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                          "gather_model_bytes": int(by_gather),
                          "frac_gather_model": round(by_gather / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)}
        tr = traffic_of.get((name, g))
        rec["traffic"] = tr
        if tr:
            rec["traffic_over_least"] = round(tr / by, 2)
        kernels.append(rec)
    dom = kernels[0]
    roofline = {"kernel": f"{dom['kernel']} (GQA {dom['gqa']})", "bound": dom["bound"],
                "achieved": dom["achieved"], "peak": dom["peak"], "unit": dom["unit"], "frac": dom["frac"],
                "traffic": dom.get("traffic"), "traffic_source": traffic_source}
    if "hbm" in dom:
        roofline["hbm"] = dom["hbm"]

    per_gqa = []
    for g in groups:
        parts = {nm: ms for (nm, gg), ms in kern.items() if gg == g}
        fwd = parts.get("selattn_fwd_main", 0) + parts.get("selattn_fwd_reduce", 0)
        bwd = sum(ms for nm, ms in parts.items() if nm.startswith("selattn_bwd"))
        tot = fwd + bwd + parts.get("index_build", 0)
        per_gqa.append({"gqa": g, "hq": hkv * g, "index_ms": round(parts.get("index_build", 0), 4),
                        "fwd_ms": round(fwd, 4), "bwd_ms": round(bwd, 4),
                        "tflops": round(flops_g[g] / 1e12 / (tot * 1e-3), 2),
                        "mfma_frac": round(flops_g[g] / 1e12 / (tot * 1e-3) / MFMA_PEAK_TFLOPS, 4),
                        **peak_mem[g]})
    # the binding roofline of the whole step: bytes through the fabric.  least = sum of the kernels' least bytes,
    # measured = sum of the counter figures (when the committed summary matches this tree)
    least_total = sum(r.get("hbm", {}).get("least_bytes", r.get("algo_bytes", 0)) for r in kernels)
    # (the index build has no line of its own in the counter summary: its few hundredths of a GB enter with their
    # algorithmic figure)
    with_bytes = [r for r in kernels if "algo_bytes" in r]
    big = [r for r in with_bytes if r["kernel"] != "index_build"]
    meas_total = (sum(r["traffic"] if r.get("traffic") else r["algo_bytes"] for r in with_bytes)
                  if big and all(r.get("traffic") for r in big) else None)

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
        "least_bytes_whole_step": int(least_total),
        "measured_bytes_whole_step": meas_total,
        "hbm_frac_whole_step": (round(meas_total / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)
                                if meas_total else None),
        "hbm_frac_whole_step_least_bytes": round(least_total / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
        # what the step could reach if every kernel moved only its least bytes at the full HBM peak: the ceiling of a
        # design that keeps one partial row per (query, block, head) in HBM
        "design_ceiling_mfma_frac": round(total_tflop / (least_total / (HBM_PEAK_GBS * 1e9)) / MFMA_PEAK_TFLOPS, 4),
        "roofline": roofline,
        "per_gqa": per_gqa,
        "kernels": kernels,
    }
    if not args.no_cpu_baseline and args.workload == "c1":
        out["cpu_baseline"] = cpu_baseline(d, bk, topk, hkv, n, p_key // hkv, args.cpu_seq_len)
        out["parity_sample"] = parity_sample(run_g, data, max(groups), idx_cpu, bk, n, dtype)
        # the same shape on the GPU, for the speed-up at equal work
        s0 = 4096
        q0, k0, v0 = (x.to(dev) for x in make_qkv(s0, hkv, hkv, d, dtype, seed=0, with_do=False))
        cu0 = torch.tensor([0, s0], dtype=torch.int32, device=dev)
        idx0 = make_topk_idx([0, s0], hkv, bk, topk, seed=1).to(dev)
        for _ in range(3):
            _topk_sparse_attention_fwd_opt(q0, k0, v0, idx0, bk, cu0, cu0, s0, s0, scale)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(20):
            _topk_sparse_attention_fwd_opt(q0, k0, v0, idx0, bk, cu0, cu0, s0, s0, scale)
        torch.cuda.synchronize()
        gpu0 = (time.perf_counter() - t0) * 1e3 / 20
        out["cpu_baseline"]["gpu_ms_same_shape"] = round(gpu0, 4)
        out["cpu_baseline"]["speedup_same_shape"] = round(out["cpu_baseline"]["ms"] / gpu0, 1)
        g1 = [r for r in per_gqa if r["gqa"] == 1]
        if g1:
            gpu1 = g1[0]["index_ms"] + g1[0]["fwd_ms"] + g1[0]["bwd_ms"]
            out["cpu_baseline"]["headline_extrapolated"]["speedup_gqa1"] = round(
                out["cpu_baseline"]["headline_extrapolated"]["gqa1_fwd_bwd_ms"] / gpu1, 0)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
