"""ctypes binding of libnsa_hip.so (the C ABI declared in include/nsa_hip.h).

There is no fallback: if the library is missing every op raises.  Build it with
`python -m nsa_amd.build` (hipcc, gfx950).
"""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libnsa_hip.so")

NSA_BF16, NSA_F32, NSA_F16 = 0, 1, 2
GATE_IDENTITY, GATE_SIGMOID = 0, 1

_P, _I, _L, _F = C.c_void_p, C.c_int, C.c_int64, C.c_float

# name -> (restype, argtypes); mirrors include/nsa_hip.h one to one
SIGNATURES = {
    "nsa_version": (_I, []),
    "nsa_last_error_string": (C.c_char_p, []),
    "nsa_transposed_offset": (_I, [_I, _I]),
    "nsa_transposed_cols": (_I, [_I, _I]),
    "nsa_compress_fwd": (_I, [_P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _P]),
    "nsa_compress_kv_fwd": (_I, [_P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _I, _P]),
    "nsa_compress_bwd": (_I, [_P] * 8 + [_I] * 8 + [_P]),
    "nsa_transpose_fwd": (_I, [_P, _P, _P, _I, _I, _I, _L, _L, _I, _I, _P]),
    "nsa_cmp_attn_select_fwd": (_I, [_P, _P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _L, _L, _I,
                                     _I, _I, _I, _I, _I, _I, _I, _I, _I, _F, _I, _I, _I, _P]),
    "nsa_cmp_attn_fwd": (_I, [_P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _L, _L, _I, _I, _I, _F, _I, _I, _P]),
    "nsa_cmp_attn_gate_fwd": (_I, [_P] * 11 + [_I, _I, _I, _I, _I, _I, _L, _L, _I, _I, _I, _F, _I, _I, _P]),
    "nsa_cmp_select_single_pass": (_I, [_I] * 10),
    "nsa_cmp_pack_chunks": (_I, [_I, _I]),
    "nsa_cmp_pack_fwd": (_I, [_P] * 4 + [_I] * 5 + [_L] * 4 + [_I, _I, _P]),
    "nsa_cmp_select_fwd": (_I, [_P] * 4 + [_I] + [_P] * 10 + [_I] * 6 + [_L, _L] + [_I] * 11 + [_F] + [_I] * 4 + [_P]),
    "nsa_block_select_fwd": (_I, [_P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _L, _L, _I, _I, _I, _I, _I, _I,
                                  _I, _I, _I, _P]),
    "nsa_gate_fwd": (_I, [_P, _P, _P, _P, _L, _I, _I, _P]),
    "nsa_gate_bwd": (_I, [_P] * 6 + [_L, _I, _I, _P]),
    "nsa_gate_combine_fwd": (_I, [_P] * 5 + [_L, _I, _I, _I, _P]),
    "nsa_gate_combine_bwd": (_I, [_P] * 10 + [_L, _I, _I, _I, _P]),
    "nsa_swa_fwd": (_I, [_P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _I, _F, _I, _P]),
    "nsa_slc_combine_fwd": (_I, [_P, _P, _P, _P, _P, _P, _P, _P, _L, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I,
                                 _I, _I, _I, _I, _F, _I, _I, _I, _P, _L, _P]),
    "nsa_slc_workspace_bytes": (_L, [_I, _I, _I, _I, _I, _I, _I, _I]),
    "nsa_slc_partials_fwd": (_I, [_P] * 6 + [_I] * 9 + [_F, _I, _I, _P, _L, _P]),
    "nsa_swa_merge_fwd": (_I, [_P] * 6 + [_L, _P, _P, _P] + [_I] * 10 + [_F, _I, _I, _P, _P, _P, _P, _P, _L, _P]),
    "nsa_slc_swa_fused_workspace_bytes": (_L, [_I] * 10),
    "nsa_slc_swa_fused_fwd": (_I, [_P] * 8 + [_L, _P, _P, _P] + [_I] * 10 + [_F, _I, _I, _I, _P, _P, _P, _P, _P, _L, _P]),
    "nsa_cmp_attn_bwd_workspace_bytes": (_L, [_I] * 6),
    "nsa_cmp_attn_bwd": (_I, [_P] * 10 + [_I] * 9 + [_F, _I, _I, _P, _P, _P, _P, _L, _P]),
    "nsa_slc_swa_bwd_workspace_bytes": (_L, [_I] * 9),
    "nsa_slc_swa_bwd_slab_workspace_bytes": (_L, [_I] * 10),
    "nsa_slc_swa_bwd": (_I, [_P] * 16 + [_I] * 9 + [_F, _I, _I, _P, _P, _P, _P, _P, _L, _P]),
    "nsa_decode_max_compressed": (_I, []),
    "nsa_decode_split_max_compressed": (_I, []),
    "nsa_decode_step": (_I, [_P] * 9 + [_I] * 15 + [_F, _I, _I, _P]),
    "nsa_qkv_rope": (_I, [_P] * 8 + [_I, _L] + [_I] * 14 + [_P]),
    "nsa_decode_append": (_I, [_P] * 7 + [_I] * 9 + [_P]),
    "nsa_decode_step_paged": (_I, [_P] * 4 + [_I] + [_P] * 6 + [_I] * 14 + [_F, _I, _I, _P]),
    "nsa_decode_split_workspace_bytes": (_L, [_I] * 5),
    "nsa_decode_split_pooled_workspace_bytes": (_L, [_I] * 8),
    "nsa_decode_step_split": (_I, [_P] * 4 + [_I] + [_P] * 6 + [_I] * 15 + [_F, _I, _I, _I, _P, _L, _P]),
    "nsa_decode_split_static_bytes": (_L, []),
    "nsa_decode_step_split_static": (_I, [_P] * 4 + [_I] + [_P] * 6 + [_I] * 15 + [_F, _I, _I, _I, _P]),
    "nsa_decode_append_paged": (_I, [_P] * 5 + [_I] + [_P] * 3 + [_I] * 8 + [_P]),
}

_lib = None


class NSALibraryError(RuntimeError):
    pass


def load():
    """Loads the shared library once; raises NSALibraryError when it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise NSALibraryError(
            "libnsa_hip.so not found at %s - run `python -m nsa_amd.build` (needs hipcc). "
            "There is no CPU or PyTorch fallback for the NSA kernels." % LIB_PATH)
    lib = C.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def check(rc: int, what: str):
    if rc == 0:
        return
    msg = load().nsa_last_error_string().decode("utf-8", "replace")
    if rc in (-1,):
        raise ValueError("%s: %s" % (what, msg))
    if rc == -2:
        raise NotImplementedError("%s: %s" % (what, msg))
    raise RuntimeError("%s failed (%d): %s" % (what, rc, msg))
