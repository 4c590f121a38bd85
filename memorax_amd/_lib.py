"""ctypes loader for libmemorax_amd.so (the C ABI declared in include/memorax_amd.h).

There is no CPU fallback: if the library is missing, or a call returns a
non-zero status, a RuntimeError is raised.
"""
from __future__ import annotations

import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "csrc", "libmemorax_amd.so")

MRX_F32, MRX_BF16, MRX_C64 = 0, 1, 2
MRX_DONE_U8, MRX_DONE_F32 = 0, 1
MRX_FMAP_NONE, MRX_FMAP_ELU1 = 0, 1
MRX_A_TIME_INVARIANT_SUM_DA = 2
MRX_FACTORS_AUTO, MRX_FACTORS_PARALLEL, MRX_FACTORS_INLINE = 0, 1, 2
MRX_RESETS_AUTO, MRX_RESETS_PASSES, MRX_RESETS_MERGED = 0, 1, 2
MRX_NOALLOC_SCRATCH_BYTES = 32 << 20

_P = ctypes.c_void_p
_I = ctypes.c_int
_L = ctypes.c_int64

# name -> (restype, argtypes); mirrors include/memorax_amd.h one to one
SIGNATURES = {
    "mrx_status_string": (ctypes.c_char_p, [_I]),
    "mrx_version": (_I, []),
    "mrx_init": (_I, [_I]),
    "mrx_chunk_size": (_L, [_I]),
    "mrx_delta_chunk_size": (_L, [_I]),
    "mrx_linear_scan_fwd": (_I, [_P] * 9 + [_L] * 3 + [_I] * 3),
    "mrx_linear_scan_bwd": (_I, [_P] * 10 + [_L] * 3 + [_I] * 3),
    "mrx_linear_attn_fwd": (_I, [_P] * 9 + [_L] * 5 + [_I] * 3),
    "mrx_linear_attn_bwd": (_I, [_P] * 13 + [_L] * 5 + [_I] * 3),
    "mrx_linear_attn_fwd_chunk_parallel": (_I, [_P] * 9 + [_L] * 5 + [_I] * 3),
    "mrx_linear_attn_bwd_chunk_parallel": (_I, [_P] * 13 + [_L] * 5 + [_I] * 3),
    "mrx_linear_attn_chunk_parallel_pays": (_I, [_L] * 3 + [_I]),
    "mrx_linear_attn_norm_fwd": (_I, [_P] * 14 + [_L] * 5 + [_I] * 3 + [ctypes.c_float]),
    "mrx_linear_attn_norm_bwd": (_I, [_P] * 19 + [_L] * 5 + [_I] * 3 + [ctypes.c_float]),
    "mrx_delta_rule_fwd": (_I, [_P] * 11 + [_L] * 5 + [_I] * 4),
    "mrx_delta_rule_fwd_noalloc": (_I, [_P] * 9 + [_L] * 5 + [_I] * 2),
    "mrx_delta_rule_bwd": (_I, [_P] * 15 + [_L] * 5 + [_I] * 3),
    "mrx_deltanet_fwd": (_I, [_P] * 11 + [_L] * 5 + [_I] * 4),
    "mrx_deltanet_bwd": (_I, [_P] * 15 + [_L] * 5 + [_I] * 3),
    "mrx_linear_scan_last": (_I, [_P] * 6 + [_L] * 4 + [_I] * 2),
    "mrx_mingru_scan_fwd": (_I, [_P] * 9 + [_L] * 3 + [_I] * 2),
    "mrx_mingru_scan_bwd": (_I, [_P] * 11 + [_L] * 3 + [_I] * 2),
    "mrx_gated_linear_attn_fwd": (_I, [_P] * 10 + [_L] * 5 + [_I] * 3),
    "mrx_gated_linear_attn_bwd": (_I, [_P] * 15 + [_L] * 5 + [_I] * 3),
    "mrx_linear_attn_step": (_I, [_P] * 10 + [_L] * 4 + [_I] * 3 + [ctypes.c_float]),
    "mrx_delta_rule_step": (_I, [_P] * 9 + [_L] * 4 + [_I] * 2),
    "mrx_gated_linear_attn_step": (_I, [_P] * 9 + [_L] * 4 + [_I] * 3),
    "mrx_mlstm_gates_fwd": (_I, [_P] * 8 + [_L] * 3 + [_I, ctypes.c_float]),
    "mrx_mlstm_gates_bwd": (_I, [_P] * 12 + [_L] * 3 + [_I, ctypes.c_float]),
    "mrx_layer_norm_fwd": (_I, [_P] * 5 + [_L] * 2 + [_I, _I, ctypes.c_float]),
    "mrx_layer_norm_bwd": (_I, [_P] * 9 + [_L] * 2 + [_I, _I, ctypes.c_float]),
    "mrx_silu_gate_fwd": (_I, [_P] * 4 + [_L, _I]),
    "mrx_silu_gate_bwd": (_I, [_P] * 6 + [_L, _I]),
    "mrx_rms_norm_fwd": (_I, [_P] * 4 + [_L] * 2 + [_I, _I, ctypes.c_float]),
    "mrx_rms_norm_bwd": (_I, [_P] * 8 + [_L] * 2 + [_I, _I, ctypes.c_float]),
}

_lib = None


def load():
    """Load the shared library once and attach the prototypes."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} not found: build it with memorax_amd/csrc/build.sh "
            "(memorax_amd has no CPU fallback)")
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the ABI is incomplete
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def check(status: int, what: str) -> None:
    if status != 0:
        msg = load().mrx_status_string(status).decode()
        raise RuntimeError(f"{what} failed: {msg} (status {status})")
