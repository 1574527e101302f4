"""CPU-side checks of the C-ABI library: it loads, exports every symbol that
include/cera_hip.h declares, and fails loudly (no fallback) without a GPU."""
import ctypes
import re
from pathlib import Path

import pytest

from cera_amd import _build, hip_api

ROOT = Path(__file__).resolve().parent.parent


def _declared_symbols():
    text = (ROOT / "include" / "cera_hip.h").read_text()
    return sorted(set(re.findall(r"\b(cera_hip_[a-z0-9_]+)\s*\(", text)))


def test_header_and_binding_agree():
    assert _declared_symbols() == sorted(hip_api.SYMBOLS)


def test_library_exports_every_declared_symbol():
    assert _build.HIP_LIB.exists(), "libcera_hip.so missing: run __graft_entry__.build()"
    lib = ctypes.CDLL(str(_build.HIP_LIB))
    missing = [s for s in _declared_symbols() if not hasattr(lib, s)]
    assert not missing, missing


def test_no_gpu_is_a_loud_error_not_a_fallback():
    lib = hip_api.load_library()
    h = ctypes.c_void_p()
    st = lib.cera_hip_ctx_create(0, None, ctypes.byref(h))
    if st == 0:          # running on a GPU box: nothing to check here
        lib.cera_hip_ctx_destroy(h)
        pytest.skip("a GPU is present")
    assert st == 1 and not h.value
    assert b"HIP" in lib.cera_hip_last_error(None) or b"device" in lib.cera_hip_last_error(None)
    with pytest.raises(hip_api.HipError):
        hip_api.Context(0)


def test_product_never_imports_the_oracle():
    """Nothing under cera_amd/ may reference oracle/ (the oracle is a checker only)."""
    for p in (ROOT / "cera_amd").rglob("*"):
        if p.suffix in {".py", ".hip", ".hip.h", ".h", ".cpp"}:
            t = p.read_text()
            assert "oracle" not in t.replace("gpu_transformer_parity", ""), p
