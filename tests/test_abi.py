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


def test_edge_shapes_are_rejected_with_a_message():
    """Empty and unsupported shapes: a negative status and a readable reason, never a launch."""
    L = ffi.lib()
    E = lambda: L.cacti_hip_last_error().decode()
    assert L.cacti_hip_rms_norm_fwd(0, 64, 16, 16, 1e-6, 16, None) == -1                  # no rows
    assert L.cacti_hip_rms_norm_bwd(4, 64, 16, 16, 1e-6, 16, 16, 0, 16, 0, 16, 8, None) == -1
    assert "workspace" in E()                                                             # too small
    assert L.cacti_hip_gemm_f16(0, 0, 0, 8, 8, 1.0, 16, 8, 16, 8, 0.0, 16, 8, None) == -1  # M = 0
    assert L.cacti_hip_gemm_f16(0, 0, 8, 8, 8, 1.0, 16, 4, 16, 8, 0.0, 16, 8, None) == -1  # lda < K
    assert "leading dimension" in E()
    # triangular modes need the square operand they describe
    assert L.cacti_hip_gemm_f16_strided_batched_tri(0, 1, 2, 16, 8, 4, 1.0, 16, 8, 4, 16, 8, 4, 0.0,
                                                    16, 16, 8, 1, None) == -1
    assert "tri=1" in E()
    assert L.cacti_hip_causal_softmax_fwd(12, 2, 16, 16, None) == -2                      # S % 8 != 0
    assert L.cacti_hip_rope_fwd(4, 2, 7, 16, 16, 16, 16, None) < 0                         # odd head dim
    assert L.cacti_hip_softmax_ce_bwd(0, 8, 16, 16, 16, 16, 0, None) == -1
    assert L.cacti_hip_embed_fwd(8, 8, 16, 0, 16, 16, 16, None) == -1                      # no positions
