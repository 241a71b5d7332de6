"""The C-ABI library loads and exports every symbol the header declares (no GPU calls)."""
import ctypes
import os
import re

from cacti_amd import ffi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _header_symbols():
    syms = set()
    for h in ("cacti_gpu_hip_ffi.h", "cacti_hip_runtime.h"):
        txt = open(os.path.join(ROOT, "include", h)).read()
        txt = re.sub(r"/\*.*?\*/", "", txt, flags=re.S)
        syms |= set(re.findall(r"\b(cacti_\w+)\s*\(", txt))
    return sorted(syms)


def test_library_exports_every_declared_symbol():
    syms = _header_symbols()
    assert len(syms) >= 40
    L = ctypes.CDLL(ffi.LIB_PATH)
    missing = [s for s in syms if not hasattr(L, s)]
    assert not missing, missing


def test_python_binding_covers_the_header():
    assert sorted(ffi.SIGNATURES) == _header_symbols()
    ffi.lib()


def test_argument_validation_needs_no_gpu():
    """Shape/pointer checks run before any HIP call, so they are testable here."""
    L = ffi.lib()
    rc = L.cacti_hip_rms_norm_fwd(4, 12, 16, 16, 1e-6, 16, None)   # D % 8 != 0
    assert rc == -2 and b"D % 8" in L.cacti_hip_last_error()
    rc = L.cacti_hip_gemm_f16(0, 0, 8, 8, 8, 1.0, 16, 8, 16, 8, 0.5, 16, 8, None)
    assert rc == -1 and b"beta" in L.cacti_hip_last_error()
    rc = L.cacti_hip_silu_gate_fwd(16, None, None, None, None)
    assert rc == -1
    assert L.cacti_hip_rms_norm_bwd_workspace(2048, 3200) == 256 * 3200 * 4
