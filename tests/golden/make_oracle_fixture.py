"""Writes tests/golden/selattn_small.npz: inputs and outputs of the CPU oracle on one small ragged case.

The reference holds no golden vectors, fixtures or CPU path, so this file is NOT a vector of the reference: it is
the frozen output of this build's own oracle (which is pinned against closed forms, dense softmax, autograd and
finite differences by tests/test_oracle_*.py).  Its purpose is to catch drift: an accidental change of the oracle
or of the seeded input generators shows up as a mismatch with the committed file.

    python tests/golden/make_oracle_fixture.py
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from oracle import selattn as orc                      # noqa: E402
from synth_inputs import make_qkv, make_topk_idx       # noqa: E402

CU, HQ, HKV, D, BK, T = [0, 70, 71, 200], 2, 1, 64, 32, 4


def compute():
    q, k, v, do = make_qkv(CU[-1], HQ, HKV, D, torch.bfloat16, seed=5)
    topk = make_topk_idx(CU, HKV, BK, T, seed=6)
    o, lse, dq, dk, dv = orc.selected_attention_grads_ref(q.float(), k.float(), v.float(), topk, BK, CU, do.float())
    cu_blocks, counts, starts, sel_tokens, slot_of = orc.build_index_ref(topk, CU, BK)
    # inputs as the raw 16-bit patterns of their bf16 values (exact, half the size of fp32)
    bits = lambda t: t.view(torch.int16).numpy()
    return dict(q_bf16=bits(q), k_bf16=bits(k), v_bf16=bits(v), do_bf16=bits(do),
                topk=topk.numpy(), o=o.numpy(), lse=lse.numpy(), dq=dq.numpy(), dk=dk.numpy(), dv=dv.numpy(),
                cu_blocks=np.asarray(cu_blocks), counts=np.asarray(counts), starts=np.asarray(starts),
                sel_tokens=np.asarray(sel_tokens), slot_of=np.asarray(slot_of))


if __name__ == "__main__":
    out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "selattn_small.npz")
    np.savez_compressed(out, **compute())
    print(out, os.path.getsize(out), "bytes")
