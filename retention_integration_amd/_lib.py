"""ctypes binding of libpower_retention_hip.so (C ABI: include/power_retention_hip.h).

There is no fallback: if the library has not been built, or a call is rejected, an exception is
raised.  Build with ``python retention_integration_amd/csrc/build.py``.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_float, c_int, c_int64, c_size_t, c_void_p

import torch

LIB_NAME = "libpower_retention_hip.so"
LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), LIB_NAME)

PR_BF16, PR_F16, PR_F32 = 0, 1, 2
DTYPES = {torch.bfloat16: PR_BF16, torch.float16: PR_F16, torch.float32: PR_F32}

_P, _I, _F = c_void_p, c_int, c_float

# name -> (restype, argtypes); mirrors include/power_retention_hip.h declaration by declaration
SIGNATURES = {
    "pr_abi_version": (c_int, []),
    "pr_set_gate_skipping": (None, [_I]),
    "pr_get_gate_skipping": (c_int, []),
    "pr_last_error": (c_char_p, []),
    "pr_expanded_dim": (c_int, [_I, _I]),
    "pr_attention_fwd": (c_int, [_P] * 7 + [_I] * 6 + [_F, _I, _I, _I, _P]),
    "pr_attention_bwd": (c_int, [_P] * 13 + [_I] * 6 + [_F, _I, _I, _P]),
    "pr_update_state_fwd": (c_int, [_P] * 5 + [_I] * 7 + [_P]),
    "pr_update_state_bwd": (c_int, [_P] * 10 + [_I] * 8 + [_P]),
    "pr_discumsum_fwd": (c_int, [_P] * 3 + [_I] * 4 + [c_int64, _I, _P]),
    "pr_discumsum_bwd_workspace": (c_size_t, [_I, _I, _I, c_int64, _I]),
    "pr_discumsum_bwd": (c_int, [_P] * 6 + [_I] * 4 + [c_int64, _I, _P]),
    "pr_query_state_fwd": (c_int, [_P] * 9 + [_I] * 6 + [_F, _I, _I, _I, _I, _P]),
    "pr_query_state_bwd_workspace": (c_size_t, [_I] * 6),
    "pr_query_state_bwd": (c_int, [_P] * 16 + [_I] * 6 + [_F, _I, _I, _I, _I, _I, _P]),
    "pr_chunk_prep_fwd": (c_int, [_P] * 8 + [_I] * 7 + [_P]),
    "pr_chunk_fwd_supported": (c_int, [_I] * 3),
    "pr_chunk_fwd": (c_int, [_P] * 12 + [_I] * 6 + [_F, _I, _I, _I, _P]),
    "pr_chunk_bwd_dq_supported": (c_int, [_I] * 3),
    "pr_chunk_bwd_dq": (c_int, [_P] * 17 + [_I] * 6 + [_F, _I, _I, _I, _P]),
    "pr_gate_cumsum": (c_int, [_P] * 2 + [_I] * 3 + [_P]),
    "pr_state_scan_fwd": (c_int, [_P] * 9 + [_I] * 4 + [c_int64, c_int64, _I, _I, _P]),
    "pr_state_chain_supported": (c_int, [_I] * 6),
    "pr_update_state_scan_fwd": (c_int, [_P] * 5 + [_I] * 7 + [_P]),
    "pr_query_state_scan_bwd_workspace": (c_size_t, [_I] * 7),
    "pr_query_state_scan_bwd": (c_int, [_P] * 17 + [_I] * 6 + [_F, _I, _I, _P]),
    "pr_state_scan_bwd_workspace": (c_size_t, [_I] * 3 + [c_int64, c_int64]),
    "pr_state_scan_bwd": (c_int, [_P] * 13 + [_I] * 4 + [c_int64, c_int64, _I, _I, _P]),
    "pr_chunk_attention_bwd": (c_int, [_P] * 18 + [_I] * 5 + [_F, _I, _I, _I, _P]),
    "pr_chunk_gate_scan_bwd": (c_int, [_P] * 5 + [_I] * 5 + [_P]),
    "pr_decode_step_workspace": (c_size_t, [_I] * 5),
    "pr_decode_step": (c_int, [_P] * 14 + [_I] * 5 + [_F, _I, _I, _I, _P]),
    "pr_cache_append": (c_int, [_P] * 7 + [_I] * 7 + [_P]),
    "pr_cache_attention_fwd": (c_int, [_P] * 7 + [_I] * 7 + [_F, _I, _I, _I, _P]),
    "pr_decode_step_noalloc_max_workspace": (c_size_t, []),
    "pr_decode_step_noalloc": (c_int, [_P] * 13 + [_I] * 5 + [_F, _I, _I, _I, _P]),
    "pr_set_launch_hook": (None, [_P, _P]),
}

# signature of the per-kernel hook: (kernel name, phase 0 / 1, stream, user pointer)
LAUNCH_HOOK = ctypes.CFUNCTYPE(None, c_char_p, c_int, c_void_p, c_void_p)

_lib = None


class PowerRetentionLibraryError(RuntimeError):
    pass


def load():
    """Load the shared library (once) and declare every entry point."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise PowerRetentionLibraryError(
            f"{LIB_PATH} is missing: the HIP kernels have not been built "
            "(run `python retention_integration_amd/csrc/build.py`); there is no fallback path")
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the library does not export it
        fn.restype, fn.argtypes = res, args
    _lib = lib
    return lib


def check(rc: int, what: str):
    if rc != 0:
        msg = load().pr_last_error().decode("utf-8", "replace")
        raise PowerRetentionLibraryError(f"{what} failed (code {rc}): {msg}")


def ptr(t):
    return None if t is None else t.data_ptr()


def stream():
    return torch.cuda.current_stream().cuda_stream


def dtype_code(dt):
    try:
        return DTYPES[dt]
    except KeyError:
        raise TypeError(f"unsupported dtype {dt}") from None
