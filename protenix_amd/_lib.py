"""ctypes binding of libprotenix_amd.so (declarations: include/protenix_amd.h).

The library is loaded from this directory.  If it has not been built yet it is
built once with hipcc (``protenix_amd.build``); if that is impossible the import
of any op fails loudly - there is no fallback implementation.
"""
from __future__ import annotations

import ctypes
import os
import threading

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libprotenix_amd.so")

PTX_F32, PTX_BF16, PTX_MIXED, PTX_F16 = 0, 1, 2, 3
ABI_VERSION = 3

_p = ctypes.c_void_p
_i = ctypes.c_int
_l = ctypes.c_int64
_f = ctypes.c_float

# name -> (restype, argtypes); mirrors include/protenix_amd.h one to one
SIGNATURES = {
    "ptx_version": (_i, []),
    "ptx_last_error_string": (ctypes.c_char_p, []),
    "ptx_key_pitch": (_i, [_i]),
    "ptx_trimul_operand_elems": (_l, [_i, _i]),
    "ptx_triattn_kv_elems": (_l, [_i, _i]),
    "ptx_triattn_bias_elems": (_l, [_i, _i]),
    "ptx_layernorm_fwd": (_i, [_p, _p, _p, _p, _p, _p, _l, _i, _f, _i, _p]),
    "ptx_layernorm_bwd_workspace_elems": (_l, [_l, _i]),
    "ptx_layernorm_bwd": (_i, [_p] * 9 + [_l, _i, _i, _p]),
    "ptx_layernorm_bwd_static": (_i, [_p] * 8 + [_l, _i, _i, _p]),
    "ptx_trimul_project": (_i, [_p] * 10 + [_i, _i, _i, _i, _i, _f, _i, _p]),
    "ptx_trimul_contract": (_i, [_p, _p, _p, _i, _i, _i, _i, _p]),
    "ptx_trimul_output": (_i, [_p] * 9 + [_i, _i, _i, _i, _f, _i, _p]),
    "ptx_triangle_multiplicative_update_workspace_elems": (_l, [_i, _i]),
    "ptx_triangle_multiplicative_update": (_i, [_p, _i] + [_p] * 11 + [_i, _i, _i, _i, _f, _i, _p]),
    "ptx_triattn_project": (_i, [_p] * 13 + [_i, _i, _i, _i, _i, _i, _f, _i, _p]),
    "ptx_triattn_fwd": (_i, [_p] * 7 + [_i, _i, _i, _i, _i, _f, _i, _p]),
    "ptx_triattn_fwd_rows": (_i, [_p] * 7 + [_i, _i, _i, _i, _i, _f, _i, _i, _i, _i, _p]),
    "ptx_triattn_output": (_i, [_p, _p, _p, _p, _i, _i, _i, _i, _i, _p]),
    "ptx_triattn_core_workspace_elems": (_l, [_i, _i, _i]),
    "ptx_triattn_core_fwd": (_i, [_p] * 8 + [_i, _i, _i, _i, _i, _i, _p]),
    "ptx_triattn_core_bwd": (_i, [_p] * 13 + [_i, _i, _i, _i, _i, _i, _p]),
    "ptx_triattn_gate_output": (_i, [_p] * 7 + [_i, _i, _i, _i, _i, _f, _i, _p]),
    "ptx_transition_packed_elems": (_l, [_i, _i]),
    "ptx_transition_pack": (_i, [_p, _p, _p, _p, _i, _i, _i, _p]),
    "ptx_transition_fwd": (_i, [_p] * 5 + [_l, _i, _i, _i, _f, _i, _p]),
    "ptx_triattn_output_transition_packed_elems": (_l, [_i]),
    "ptx_triattn_output_transition_pack": (_i, [_p] * 6 + [_i, _i, _p]),
    "ptx_triattn_output_transition_fwd": (_i, [_p] * 8 + [_i, _i, _i, _i, _i, _f, _f, _p, _p, _p, _p, _i, _i,
                                               _f, _i, _p]),
    "ptx_transition_pair_bias_fwd": (_i, [_p] * 5 + [_l, _i, _i, _i, _f, _p, _p, _p, _p, _i, _i, _f, _i, _p]),
    "ptx_linear_fwd": (_i, [_p, _p, _p, _i, _p, _p, _p, _i, _l, _i, _i, _i, _i, _p]),
    "ptx_swiglu_fwd": (_i, [_p, _p, _p, _p, _i, _i, _i, _i, _p]),
    "ptx_single_attention_fwd": (_i, [_p, _p, _p, _p, _p, _i, _p, _i, _i, _i, _l, _l, _l, _f, _i, _p]),
    "ptx_pair_bias_fwd": (_i, [_p] * 5 + [_i, _i, _i, _i, _f, _i, _p]),
    "ptx_hbm_stream": (_i, [_p, _p, _l, _i, _p]),
}

_lock = threading.Lock()
_lib = None


def load() -> ctypes.CDLL:
    """Returns the loaded library, building it first if it does not exist."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        if not os.path.exists(LIB_PATH):
            from . import build as _build

            _build.build()
        lib = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)      # AttributeError if the build is stale
            fn.restype = res
            fn.argtypes = args
        if lib.ptx_version() != ABI_VERSION:
            raise RuntimeError(
                f"{LIB_PATH}: ABI version {lib.ptx_version()} != expected {ABI_VERSION}; rebuild "
                "with `python -m protenix_amd.build`")
        _lib = lib
    return _lib


def check(rc: int, what: str) -> None:
    if rc != 0:
        msg = load().ptx_last_error_string().decode("utf-8", "replace")
        kind = {1: "bad argument", 2: "unsupported shape", 3: "launch failure"}.get(rc, "error")
        raise RuntimeError(f"{what}: {kind} ({rc}): {msg}")
