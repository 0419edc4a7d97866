"""The C-ABI library loads without a GPU and exports every symbol include/fsa_hip.h declares;
host-side argument checks of entry points that need no device work."""
import ctypes as C
import os
import re

import pytest

from fsa_hip import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "fsa_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(fsa_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported_and_bound():
    names = _declared()
    assert len(names) >= 20
    lib = _lib.load()
    for n in names:
        assert hasattr(lib, n), f"{n} declared in include/fsa_hip.h but not exported"
        assert n in _lib.SIGNATURES, f"{n} has no ctypes prototype"
    assert set(_lib.SIGNATURES) <= set(names)


def test_version_and_host_arithmetic():
    lib = _lib.load()
    assert lib.fsa_version() >= 210
    # tiles upper bound: ceil(N*T*g / rows) + max_blocks
    assert lib.fsa_max_tiles(65536, 16, 1, 1024, 1025) == 65536 * 16 // 1024 + 1025
    # counting path (at most 4095 blocks): one count per (kv head, block or padding bucket, tile of 4096 entries)
    assert lib.fsa_index_workspace_bytes(65536, 16, 4, 1025) >= 4 * 1026 * (65536 * 16 // 4096) * 4
    # radix path beyond that: two key and two value buffers of N*T entries per kv head
    assert lib.fsa_index_workspace_bytes(65536, 16, 4, 4097) >= 4 * 65536 * 16 * 4 * 4
    a = lib.fsa_selattn_fwd_workspace_bytes(65536, 4, 4, 128, 16, 1025)
    b = lib.fsa_selattn_fwd_workspace_bytes(65536, 16, 4, 128, 16, 1025)
    assert b > 3 * a  # partial buffers scale with the GQA group


def test_invalid_arguments_are_reported_not_launched():
    lib = _lib.load()
    rc = lib.fsa_build_tiles(None, 4, 10, 1, 128, None, None)
    assert rc == -1 and b"null" in lib.fsa_last_error()
    rc = lib.fsa_build_index(None, 0, 0, None, 1, 16, 1, 4, 64, 2, None, None, None, None, None, None, 0, None)
    assert rc == -1
    with pytest.raises(ValueError):
        _lib.check(rc, "fsa_build_index")


def test_dense_attention_refuses_row_strides_beyond_its_tile_offsets():
    """The dense kernels address a K / V tile with 32-bit lane offsets; a row stride that does not fit is an
    argument error, raised before anything is launched (fake, never dereferenced pointers)."""
    lib = _lib.load()
    fake = 0x1000
    args = dict(dtype=0, q_sn=512, q_sh=128, k_sn=1 << 26, k_sh=128, v_sn=128, v_sh=128)
    rc = lib.fsa_winattn_fwd(fake, fake, fake, args["dtype"], args["q_sn"], args["q_sh"], args["k_sn"], args["k_sh"],
                             args["v_sn"], args["v_sh"], fake, 1, 64, 64, 4, 1, 128, 16, 0.1, fake, 512, 128, fake, None)
    assert rc == -1 and b"stride" in lib.fsa_last_error()
    # backward: q, k, v, o, d_o, lse, dtype, strides of q / k (too large) / v / o / d_o, cu_seqlens, batch,
    # total_tokens, max_seqlen, Hq, Hkv, D, window, scale, dq, dk, dv, workspace
    rc = lib.fsa_winattn_bwd(fake, fake, fake, fake, fake, fake, 0, 512, 128, 1 << 26, 128, 128, 128, 512, 128, 512, 128,
                             fake, 1, 64, 64, 4, 1, 128, 16, 0.1, fake, fake, fake, fake, 1 << 40, None)
    assert rc == -1 and b"row stride too large" in lib.fsa_last_error(), lib.fsa_last_error()


def test_selected_attention_refuses_q_strides_beyond_32_bits():
    """The gathers form q / dO row addresses with 32-bit strides: a token stride of 2^31 elements is an argument
    error of the forward and the backward entry points, raised before the workspace is looked at or anything is
    launched (fake, never dereferenced pointers)."""
    lib = _lib.load()
    f = 0x1000
    big = 1 << 31
    rc = lib.fsa_selattn_fwd(f, f, f, 0, big, 128, 512, 128, 512, 128, f, 1, 1024, 4, 1, 128, 16, 64, 16, 0.1,
                             f, f, f, f, f, f, 512, 128, f, f, 1 << 40, None)
    assert rc == -1 and b"too large" in lib.fsa_last_error(), lib.fsa_last_error()
    # q, k, v, o, d_o, lse, dtype, strides of q / k / v / o (fine) and of d_o (too large), cu_seqlens, batch,
    # total_tokens, Hq, Hkv, D, topk, block_size, max_blocks, scale, index arrays, dq, dk, dv, workspace
    rc = lib.fsa_selattn_bwd(f, f, f, f, f, f, 0, 512, 128, 512, 128, 512, 128, 512, 128, big, 128,
                             f, 1, 1024, 4, 1, 128, 16, 64, 16, 0.1, f, f, f, f, f, f, f, f, f, 1 << 40, None)
    assert rc == -1 and b"too large" in lib.fsa_last_error(), lib.fsa_last_error()


def test_wrappers_refuse_cpu_tensors():
    import torch

    from fsa_hip import ops

    t = torch.zeros(1, 4, 2, dtype=torch.int32)
    with pytest.raises(RuntimeError, match="no CPU path"):
        ops.build_index(t, torch.tensor([0, 4], dtype=torch.int32), 64)


def test_every_compute_entry_point_rejects_null_pointers():
    """All-zero arguments: each entry point must answer with the invalid-argument code and a message before it
    touches a device (this runs on machines without a GPU)."""
    lib = _lib.load()
    skip = {"fsa_version", "fsa_profile_enable", "fsa_profile_count"}
    for name, (res, args) in _lib.SIGNATURES.items():
        if res is not C.c_int or name in skip:
            continue
        vals = []
        for a in args:
            if a in (C.c_void_p, C.c_char_p) or getattr(a, "__name__", "").startswith("LP_"):
                vals.append(None)
            elif a in (C.c_float, C.c_double):
                vals.append(0.0)
            else:
                vals.append(0)
        rc = getattr(lib, name)(*vals)
        assert rc == -1, (name, rc)
        assert lib.fsa_last_error(), name


def test_pad_head_dim_argument_checks():
    """fsa_native_head_dim is host arithmetic; fsa_pad_head_dim refuses bad strides / alignment / sizes before any
    launch (no device needed for either)."""
    lib = _lib.load()
    assert [lib.fsa_native_head_dim(d) for d in (0, 1, 64, 65, 128, 129, 256, 257)] == [-1, 64, 64, 128, 128, 256, 256, -1]
    f = 4096
    ok = dict(src=f, sn=96, sh=96, ds=96, dst=f, dn=128, dh=128, dd=128, rows=4, heads=1)

    def call(**kw):
        a = dict(ok, **kw)
        return lib.fsa_pad_head_dim(a["src"], a["sn"], a["sh"], a["ds"], a["dst"], a["dn"], a["dh"], a["dd"], a["rows"],
                                    a["heads"], None)

    for bad in (dict(src=None), dict(dst=None), dict(rows=0), dict(heads=0), dict(ds=0), dict(dd=2), dict(dd=126),
                dict(sn=-96), dict(sn=98), dict(dh=130), dict(src=f + 4), dict(rows=1 << 45)):
        assert call(**bad) == -1, bad
        assert b"fsa_pad_head_dim" in lib.fsa_last_error()
