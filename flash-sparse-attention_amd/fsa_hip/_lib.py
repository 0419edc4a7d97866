"""ctypes loader for libfsa_gfx950.so (the C ABI declared in include/fsa_hip.h).

The library is built in-tree by `build.py`; loading fails loudly when it is
missing - there is no fallback path.
"""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("FSA_HIP_LIBRARY") or os.path.join(_HERE, "libfsa_gfx950.so")

_lib = None

i32, i64, f32, vp, sz = C.c_int32, C.c_int64, C.c_float, C.c_void_p, C.c_size_t

# name -> (restype, argtypes); mirrors include/fsa_hip.h one to one
SIGNATURES = {
    "fsa_version": (C.c_int, []),
    "fsa_last_error": (C.c_char_p, []),
    "fsa_native_head_dim": (C.c_int, [i32]),
    "fsa_pad_head_dim": (C.c_int, [vp, i64, i64, i32, vp, i64, i64, i32, i64, i32, vp]),
    "fsa_profile_enable": (C.c_int, [C.c_int]),
    "fsa_profile_count": (C.c_int, []),
    "fsa_profile_get": (C.c_int, [C.c_int, C.c_char_p, C.c_int, C.POINTER(C.c_float)]),
    "fsa_index_workspace_bytes": (sz, [i64, i32, i32, i64]),
    "fsa_build_index": (C.c_int, [vp, i64, i64, vp, i32, i64, i32, i32, i32, i64,
                                  vp, vp, vp, vp, vp, vp, sz, vp]),
    "fsa_split_topk_blocks": (C.c_int, [vp, i64, i64, vp, i32, i64, i32, i32, i32, i32, vp, vp]),
    "fsa_build_tiles": (C.c_int, [vp, i32, i64, i32, i32, vp, vp]),
    "fsa_max_tiles": (i64, [i64, i32, i32, i32, i64]),
    "fsa_selattn_fwd_workspace_bytes": (sz, [i64, i32, i32, i32, i32, i64]),
    "fsa_selattn_fwd": (C.c_int, [vp, vp, vp, i32, i64, i64, i64, i64, i64, i64,
                                  vp, i32, i64, i32, i32, i32, i32, i32, i64, f32,
                                  vp, vp, vp, vp, vp,
                                  vp, i64, i64, vp, vp, sz, vp]),
    "fsa_selattn_bwd_workspace_bytes": (sz, [i64, i32, i32, i32, i32, i32, i64]),
    "fsa_selattn_bwd": (C.c_int, [vp, vp, vp, vp, vp, vp, i32,
                                  i64, i64, i64, i64, i64, i64, i64, i64, i64, i64,
                                  vp, i32, i64, i32, i32, i32, i32, i32, i64, f32,
                                  vp, vp, vp, vp, vp,
                                  vp, vp, vp, vp, sz, vp]),
    "fsa_cmpattn_fwd": (C.c_int, [vp, vp, vp, i32, i64, i64, i64, i64, i64, i64,
                                  vp, vp, i32, i64, i64, i32, i32, i32, i32, i32, f32,
                                  vp, i64, i64, vp, vp]),
    "fsa_cmpattn_bwd_workspace_bytes": (sz, [i64, i64, i64, i32, i32, i32, i32]),
    "fsa_cmpattn_bwd": (C.c_int, [vp, vp, vp, vp, vp, vp, i32,
                                  i64, i64, i64, i64, i64, i64, i64, i64, i64, i64,
                                  vp, vp, i32, i64, i64, i64, i32, i32, i32, i32, i32, f32,
                                  vp, vp, vp, vp, sz, vp]),
    "fsa_cmp_topk_workspace_bytes": (sz, [i64, i32, i64]),
    "fsa_cmp_topk": (C.c_int, [vp, vp, vp, i32, i64, i64, i64, i64, vp, vp, i32,
                               i64, i64, i64, i32, i32, i32, i32, i32, i32, i32, i32, i32, i32, i32, f32,
                               vp, vp, vp, sz, vp]),
    "fsa_winattn_fwd": (C.c_int, [vp, vp, vp, i32, i64, i64, i64, i64, i64, i64, vp, i32, i64, i64,
                                  i32, i32, i32, i32, f32, vp, i64, i64, vp, vp]),
    "fsa_winattn_bwd_workspace_bytes": (sz, [i64, i64, i32, i32, i32, i32, i32]),
    "fsa_winattn_bwd": (C.c_int, [vp, vp, vp, vp, vp, vp, i32,
                                  i64, i64, i64, i64, i64, i64, i64, i64, i64, i64,
                                  vp, i32, i64, i64, i32, i32, i32, i32, f32,
                                  vp, vp, vp, vp, sz, vp]),
    "fsa_rope": (C.c_int, [vp, vp, i32, i64, i64, i64, i64, vp, i32, i64, i32, i32, vp, f32, i32, i32, i32, vp]),
    "fsa_linear_compress_fwd": (C.c_int, [vp, vp, vp, i32, i64, i64, vp, vp, i32, i64, i32, i32, i32, i32,
                                          vp, vp, vp]),
    "fsa_linear_compress_bwd": (C.c_int, [vp, vp, vp, vp, i32, i64, i64, vp, vp, i32, i64, i64, i32, i32,
                                          i32, i32, vp, vp, vp, vp, vp]),
    "fsa_gate_merge_fwd": (C.c_int, [vp, vp, vp, vp, i32, i64, i32, vp, vp]),
    "fsa_gate_merge_bwd": (C.c_int, [vp, vp, vp, vp, vp, i32, i64, i32, vp, vp, vp, vp, vp]),
    "fsa_decode_workspace_bytes": (C.c_size_t, [i32, i32, i32, i32, i64]),
    "fsa_decode_cmpattn": (C.c_int, [vp, vp, vp, i32, i64, i64, i64, i64, i64, i64, vp, vp,
                                     i32, i32, i32, i32, i32, i32, f32, i32, i64, vp, vp, vp, i64, vp, sz, vp]),
    "fsa_decode_topk": (C.c_int, [vp, i64, vp, vp, vp, vp, i32, i32, i32, i32, i32, i32,
                                  i32, i32, i32, i32, i32, f32, i64, vp, vp, vp]),
    "fsa_decode_selattn": (C.c_int, [vp, vp, vp, i32, i64, i64, i64, i64, i64, i64, vp, vp, vp,
                                     i32, i32, i32, i32, i32, i32, f32, vp, vp, vp, sz, vp]),
    "fsa_decode_selattn_static": (C.c_int, [vp, vp, vp, i32, i64, i64, i64, i64, i64, i64, vp, vp, vp,
                                            i32, i32, i32, i32, i32, i32, f32, vp, vp, vp]),
}


def load():
    """Load the shared library once and attach the prototypes."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} not found: build it with `python flash-sparse-attention_amd/build.py` "
            "(hipcc, gfx950). There is no fallback implementation.")
    lib = C.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        if not hasattr(lib, name):
            continue  # reported by exported_symbols(); calling it raises AttributeError
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def exported_symbols():
    lib = load()
    return {name: hasattr(lib, name) for name in SIGNATURES}


def check(rc: int, what: str):
    """Translate the C ABI's return code into a Python exception."""
    if rc == 0:
        return
    msg = load().fsa_last_error().decode("utf-8", "replace")
    if rc < 0:
        raise ValueError(f"{what}: {msg} (code {rc})")
    raise RuntimeError(f"{what}: HIP error {rc}: {msg}")


def profile_enable(on: bool):
    load().fsa_profile_enable(1 if on else 0)


def profile_records():
    """[(label, milliseconds)] of the launches recorded since profile_enable(True)."""
    lib = load()
    out = []
    buf = C.create_string_buffer(128)
    ms = C.c_float()
    for i in range(lib.fsa_profile_count()):
        check(lib.fsa_profile_get(i, buf, 128, C.byref(ms)), "fsa_profile_get")
        out.append((buf.value.decode(), ms.value))
    return out
