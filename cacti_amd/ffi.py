"""ctypes binding of libcacti_gpu_hip_ffi.so (the C ABI in include/cacti_gpu_hip_ffi.h).

Loading fails loudly when the library has not been built: there is no CPU fallback.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libcacti_gpu_hip_ffi.so")

i64, f32, vp, ci, sz = C.c_int64, C.c_float, C.c_void_p, C.c_int, C.c_size_t
pvp = C.POINTER(C.c_void_p)

# name -> (restype, argtypes); mirrors the header one to one
SIGNATURES = {
    "cacti_hip_last_error": (C.c_char_p, []),
    "cacti_hip_device_count": (ci, [C.POINTER(ci)]),
    "cacti_hip_device_get": (ci, [C.POINTER(ci)]),
    "cacti_hip_device_set": (ci, [ci]),
    "cacti_hip_device_attribute": (ci, [ci, ci, C.POINTER(ci)]),
    "cacti_hip_device_sync": (ci, []),
    "cacti_hip_mem_get_info": (ci, [C.POINTER(sz), C.POINTER(sz)]),
    "cacti_hip_mem_alloc": (ci, [pvp, sz]),
    "cacti_hip_mem_free": (ci, [vp]),
    "cacti_hip_mem_alloc_host": (ci, [pvp, sz]),
    "cacti_hip_mem_free_host": (ci, [vp]),
    "cacti_hip_memcpy_d2h": (ci, [vp, vp, sz]),
    "cacti_hip_memcpy_async": (ci, [vp, vp, sz, vp]),
    "cacti_hip_memcpy_h2d_async": (ci, [vp, vp, sz, vp]),
    "cacti_hip_memcpy_d2h_async": (ci, [vp, vp, sz, vp]),
    "cacti_hip_memset_async": (ci, [vp, ci, sz, vp]),
    "cacti_hip_stream_create": (ci, [pvp]),
    "cacti_hip_stream_create_nonblocking": (ci, [pvp]),
    "cacti_hip_stream_destroy": (ci, [vp]),
    "cacti_hip_stream_sync": (ci, [vp]),
    "cacti_hip_stream_wait_event": (ci, [vp, vp]),
    "cacti_hip_event_create": (ci, [pvp, ci]),
    "cacti_hip_event_destroy": (ci, [vp]),
    "cacti_hip_event_record": (ci, [vp, vp]),
    "cacti_hip_event_query": (ci, [vp]),
    "cacti_hip_event_sync": (ci, [vp]),
    "cacti_hip_event_elapsed_ms": (ci, [vp, vp, C.POINTER(f32)]),
    "cacti_hip_gemm_f16": (ci, [ci, ci, i64, i64, i64, f32, vp, i64, vp, i64, f32, vp, i64, vp]),
    "cacti_hip_gemm_f16_strided_batched": (ci, [ci, ci, i64, i64, i64, i64, f32, vp, i64, i64, vp,
                                                i64, i64, f32, vp, i64, i64, vp]),
    "cacti_hip_gemm_colmajor_f16": (ci, [ci, ci, ci, ci, ci, C.POINTER(f32), vp, ci, vp, ci,
                                         C.POINTER(f32), vp, ci, vp]),
    "cacti_hip_accumulate_1d_f32": (ci, [vp, vp, i64, vp]),
    "cacti_hip_accumulate_1d_f16": (ci, [vp, vp, i64, vp]),
    "cacti_hip_accumulate_1d_u16": (ci, [vp, vp, i64, vp]),
    "cacti_hip_rms_norm_fwd": (ci, [i64, i64, vp, vp, f32, vp, vp]),
    "cacti_hip_rms_norm_bwd_workspace": (sz, [i64, i64]),
    "cacti_hip_rms_norm_bwd": (ci, [i64, i64, vp, vp, f32, vp, vp, ci, vp, ci, vp, sz, vp]),
    "cacti_hip_rope_tables": (ci, [i64, i64, vp, vp, vp]),
    "cacti_hip_rope_fwd": (ci, [i64, i64, i64, vp, vp, vp, vp, vp]),
    "cacti_hip_rope_bwd": (ci, [i64, i64, i64, vp, vp, vp, vp, ci, vp]),
    "cacti_hip_silu_gate_fwd": (ci, [i64, vp, vp, vp, vp]),
    "cacti_hip_silu_gate_bwd": (ci, [i64, vp, vp, vp, vp, ci, vp, ci, vp]),
    "cacti_hip_causal_softmax_fwd": (ci, [i64, i64, vp, vp, vp]),
    "cacti_hip_causal_softmax_bwd": (ci, [i64, i64, vp, vp, vp, vp]),
    "cacti_hip_softmax_ce_fwd": (ci, [i64, i64, vp, vp, vp, vp, vp, vp, vp]),
    "cacti_hip_softmax_ce_bwd": (ci, [i64, i64, vp, vp, vp, vp, ci, vp]),
    "cacti_hip_embed_fwd": (ci, [i64, i64, vp, i64, vp, vp, vp, vp]),
    "cacti_hip_embed_bwd": (ci, [i64, i64, i64, vp, vp, vp, ci, vp]),
    "cacti_hip_add_f16": (ci, [i64, vp, vp, vp, vp]),
    "cacti_hip_selftest_wave_reduce": (ci, [vp, vp]),
}

_lib = None


class CactiError(RuntimeError):
    def __init__(self, code, msg):
        super().__init__("cacti_gpu_hip_ffi status %d: %s" % (code, msg))
        self.code = code


def lib():
    """The loaded library; raises if it is not built (no fallback)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                "%s is missing: build it with `python -m cacti_amd.build` "
                "(hipcc --offload-arch=gfx950); there is no CPU fallback" % LIB_PATH)
        L = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


def check(rc):
    if rc != 0:
        raise CactiError(rc, lib().cacti_hip_last_error().decode("utf-8", "replace"))


def call(name, *args):
    check(getattr(lib(), name)(*args))
