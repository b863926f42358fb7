"""The C-ABI library loads without a GPU and exports every entry point that include/power_retention_hip.h declares;
the ctypes table (retention_integration_amd/_lib.py) names exactly the same set.  No kernel is launched here."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "power_retention_hip.h")
LIB = os.path.join(ROOT, "retention_integration_amd", "libpower_retention_hip.so")


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(pr_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_entry_points():
    names = declared_symbols()
    for must in ("pr_attention_fwd", "pr_attention_bwd", "pr_update_state_fwd", "pr_update_state_bwd",
                 "pr_discumsum_fwd", "pr_discumsum_bwd", "pr_query_state_fwd", "pr_query_state_bwd",
                 "pr_decode_step", "pr_last_error", "pr_abi_version"):
        assert must in names


def test_ctypes_table_matches_header():
    from retention_integration_amd import _lib
    assert sorted(_lib.SIGNATURES) == declared_symbols()


@pytest.mark.skipif(not os.path.exists(LIB), reason="library not built (python retention_integration_amd/csrc/build.py)")
def test_library_exports_every_declared_symbol():
    lib = ctypes.CDLL(LIB)
    for name in declared_symbols():
        assert hasattr(lib, name), f"{name} is declared in the header but not exported"
    lib.pr_abi_version.restype = ctypes.c_int
    assert lib.pr_abi_version() >= 1
    lib.pr_expanded_dim.restype = ctypes.c_int
    lib.pr_expanded_dim.argtypes = [ctypes.c_int, ctypes.c_int]
    assert [lib.pr_expanded_dim(d, 2) for d in (32, 64, 128)] == [768, 2560, 9216]
    # argument checks run before any launch: a bad head dimension is refused with a message
    lib.pr_update_state_fwd.restype = ctypes.c_int
    lib.pr_update_state_fwd.argtypes = [ctypes.c_void_p] * 5 + [ctypes.c_int] * 7 + [ctypes.c_void_p]
    rc = lib.pr_update_state_fwd(16, 16, 16, 16, None, 1, 16, 1, 48, 2, 0, 0, None)
    lib.pr_last_error.restype = ctypes.c_char_p
    assert rc != 0 and b"head dim" in lib.pr_last_error()
