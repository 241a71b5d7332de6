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
    "cacti_hip_primary_ctx_retain": (ci, [ci, pvp]),
    "cacti_hip_primary_ctx_release": (ci, [ci]),
    "cacti_hip_primary_ctx_set_flags": (ci, [ci, C.c_uint]),
    "cacti_hip_primary_ctx_reset": (ci, [ci]),
    "cacti_hip_stream_null": (vp, []),
    "cacti_parse_byte_size": (ci, [C.c_char_p, C.POINTER(C.c_uint64)]),
    "cacti_vmem_soft_limit": (ci, [C.c_char_p, sz, sz, C.POINTER(sz)]),
    "cacti_env_host_pagelocked": (ci, []),
    "cacti_hip_stream_wait_event": (ci, [vp, vp]),
    "cacti_hip_event_create": (ci, [pvp, ci]),
    "cacti_hip_event_destroy": (ci, [vp]),
    "cacti_hip_event_record": (ci, [vp, vp]),
    "cacti_hip_event_query": (ci, [vp]),
    "cacti_hip_event_sync": (ci, [vp]),
    "cacti_hip_event_elapsed_ms": (ci, [vp, vp, C.POINTER(f32)]),
    "cacti_hip_gemm_f16": (ci, [ci, ci, i64, i64, i64, f32, vp, i64, vp, i64, f32, vp, i64, vp]),
    "cacti_hip_gemm_f16_batched": (ci, [ci, ci, i64, i64, i64, i64, f32, vp, i64, vp, i64, f32, vp, i64, vp]),
    "cacti_hip_gemm_f16_strided_batched": (ci, [ci, ci, i64, i64, i64, i64, f32, vp, i64, i64, vp,
                                                i64, i64, f32, vp, i64, i64, vp]),
    "cacti_hip_gemm_f16_strided_batched_tri": (ci, [ci, ci, i64, i64, i64, i64, f32, vp, i64, i64,
                                                    vp, i64, i64, f32, vp, i64, i64, ci, vp]),
    "cacti_hip_gemm_colmajor_f16": (ci, [ci, ci, ci, ci, ci, C.POINTER(f32), vp, ci, vp, ci,
                                         C.POINTER(f32), vp, ci, vp]),
    "cacti_hip_accumulate_1d_f32": (ci, [vp, vp, i64, vp]),
    "cacti_hip_accumulate_1d_f16": (ci, [vp, vp, i64, vp]),
    "cacti_hip_accumulate_1d_u16": (ci, [vp, vp, i64, vp]),
    "cacti_hip_rms_norm_fwd": (ci, [i64, i64, vp, vp, f32, vp, vp]),
    "cacti_hip_add_rms_norm_fwd": (ci, [i64, i64, vp, vp, vp, f32, vp, vp, vp]),
    "cacti_hip_rms_norm_bwd_workspace": (sz, [i64, i64]),
    "cacti_hip_rms_norm_bwd": (ci, [i64, i64, vp, vp, f32, vp, vp, ci, vp, ci, vp, sz, vp]),
    "cacti_hip_rms_norm_bwd_static_max_bytes": (sz, []),
    "cacti_hip_rms_norm_bwd_static": (ci, [i64, i64, vp, vp, f32, vp, vp, ci, vp, ci, vp]),
    "cacti_hip_rope_tables": (ci, [i64, i64, vp, vp, vp]),
    "cacti_hip_rope_fwd": (ci, [i64, i64, i64, vp, vp, vp, vp, vp]),
    "cacti_hip_rope_bwd": (ci, [i64, i64, i64, vp, vp, vp, vp, ci, vp]),
    "cacti_hip_rope_fwd_pair": (ci, [i64, i64, i64, vp, vp, vp, vp, vp, vp, vp]),
    "cacti_hip_rope_bwd_pair": (ci, [i64, i64, i64, vp, vp, vp, vp, vp, ci, vp, ci, vp]),
    "cacti_hip_silu_gate_fwd": (ci, [i64, vp, vp, vp, vp]),
    "cacti_hip_silu_gate_bwd": (ci, [i64, vp, vp, vp, vp, ci, vp, ci, vp]),
    "cacti_hip_causal_softmax_fwd": (ci, [i64, i64, vp, vp, vp]),
    "cacti_hip_causal_softmax_bwd": (ci, [i64, i64, vp, vp, vp, vp]),
    "cacti_hip_mfma_probe": (ci, [ci, ci, ci, ci, i64, C.c_uint, vp, vp]),
    "cacti_hip_attention_set_exact": (ci, [ci]),
    "cacti_hip_attention_stats_bytes": (sz, [i64, i64]),
    "cacti_hip_attention_fwd": (ci, [i64, i64, i64, f32, vp, vp, vp, i64, vp, vp, vp]),
    "cacti_hip_attention_bwd_workspace": (sz, [i64, i64]),
    "cacti_hip_attention_bwd": (ci, [i64, i64, i64, f32, vp, vp, vp, vp, vp, i64, vp, vp, ci, vp, ci, vp, ci,
                                     vp, sz, vp]),
    "cacti_hip_softmax_ce_fwd": (ci, [i64, i64, vp, vp, vp, vp, vp, vp, vp]),
    "cacti_hip_softmax_ce_bwd": (ci, [i64, i64, vp, vp, vp, vp, ci, vp]),
    "cacti_hip_embed_fwd": (ci, [i64, i64, vp, i64, vp, vp, vp, vp]),
    "cacti_hip_embed_bwd": (ci, [i64, i64, i64, vp, vp, vp, ci, vp]),
    "cacti_hip_add_f16": (ci, [i64, vp, vp, vp, vp]),
    "cacti_hip_selftest_wave_reduce": (ci, [vp, vp]),
    "cacti_hip_nan_count_f16": (ci, [i64, vp, vp, vp]),
    "cacti_hip_abs_log2_hist8_f16": (ci, [i64, vp, vp, vp]),
    "cacti_hip_digests_scratch_bytes": (sz, [ci]),
    "cacti_hip_digests_f16_batch": (ci, [ci, vp, vp, vp, vp, vp]),
    "cacti_hip_online_average_scale_f16_f32": (ci, [i64, vp, vp, f32, f32, vp]),
    "cacti_hip_online_average_square_scale_f16_f32": (ci, [i64, vp, vp, f32, f32, vp]),
    "cacti_hip_online_adamw_update_f32": (ci, [i64, vp, vp, vp, f32, f32, f32, f32, vp]),
    "cacti_hip_cast_f32_f16": (ci, [i64, vp, vp, vp]),
    "cacti_hip_cast_f16_f32": (ci, [i64, vp, vp, vp]),
    "cacti_hip_row_causal_softmax_fwd": (ci, [i64, i64, i64, i64, i64, vp, vp, vp]),
    "cacti_hip_rows_norm_matmul_f16": (ci, [i64, i64, i64, vp, vp, vp, f32, vp, vp, vp, vp, vp]),
    "cacti_hip_rows_qkv_rope_cache_f16": (ci, [i64, i64, i64, vp, vp, vp, f32, vp, vp, vp, vp, vp, vp, vp, vp, vp, vp]),
    "cacti_hip_attn_decode_workspace": (sz, [i64, i64, i64, i64]),
    "cacti_hip_attn_decode_f16": (ci, [i64, i64, i64, i64, i64, f32, vp, i64, vp, vp, i64, i64, vp, i64, vp, sz, vp]),
    "cacti_hip_append_token_u16": (ci, [vp, i64, vp, i64, vp]),
    "cacti_hip_raw_cast_bf16_f16": (ci, [i64, vp, vp, vp]),
    "cacti_hip_raw_cast_bf16_f32": (ci, [i64, vp, vp, vp]),
    "cacti_hip_raw_cast_f32_bf16": (ci, [i64, vp, vp, vp]),
    "cacti_hip_raw_cast_f16_bf16": (ci, [i64, vp, vp, vp]),
    "cacti_adamw32_scalars": (ci, [ci, f32, f32, f32, f32, f32, f32, vp]),
    "cacti_hip_adamw32_scratch_bytes": (sz, [ci]),
    "cacti_hip_adamw32_step_f16_batch": (ci, [ci, vp, vp, vp, vp, vp, vp, vp, vp, vp]),
    # ---- runtime (include/cacti_hip_runtime.h)
    "cacti_ctx_create": (ci, [pvp, ci, sz, ci]),
    "cacti_ctx_destroy": (ci, [vp]),
    "cacti_ctx_stats": (ci, [vp, vp]),
    "cacti_ctx_usage_report": (ci, [vp, C.c_char_p, sz]),
    "cacti_ctx_sync": (ci, [vp]),
    "cacti_ctx_stream": (vp, [vp]),
    "cacti_ctx_set_timing": (ci, [vp, ci]),
    "cacti_ctx_set_timing_filter": (ci, [vp, C.c_char_p, ci]),
    "cacti_ctx_timing_report": (ci, [vp, C.c_char_p, sz]),
    "cacti_mempool_create": (ci, [pvp, C.c_uint64]),
    "cacti_mempool_destroy": (ci, [vp]),
    "cacti_mempool_alloc": (C.c_uint64, [vp, C.c_uint64]),
    "cacti_mempool_alloc_high": (C.c_uint64, [vp, C.c_uint64]),
    "cacti_mempool_free": (ci, [vp, C.c_uint64]),
    "cacti_mempool_stats": (ci, [vp, C.POINTER(C.c_uint64)]),
    "cacti_reset": (ci, [vp]),
    "cacti_compile": (ci, [vp]),
    "cacti_resume": (ci, [vp, C.POINTER(ci)]),
    "cacti_resume_put": (ci, [vp, ci, vp, sz]),
    "cacti_cell_bytes": (ci, [vp, ci, C.POINTER(sz)]),
    "cacti_cell_get": (ci, [vp, ci, vp, sz]),
    "cacti_log_len": (ci, [vp]),
    "cacti_log_name": (C.c_char_p, [vp, ci]),
    "cacti_llama_create": (ci, [vp, vp, pvp]),
    "cacti_llama_destroy": (ci, [vp]),
    "cacti_llama_num_params": (ci, [vp]),
    "cacti_llama_param_info": (ci, [vp, ci, C.c_char_p, sz, C.POINTER(i64), C.POINTER(i64),
                                    C.POINTER(ci), C.POINTER(ci)]),
    "cacti_llama_param_put": (ci, [vp, ci, vp, sz]),
    "cacti_llama_grad_get": (ci, [vp, ci, vp, sz]),
    "cacti_llama_digests": (ci, [vp, ci, vp, vp]),
    "cacti_tensors_dir_open": (ci, [C.c_char_p, pvp]),
    "cacti_pickle_dir_open": (ci, [C.c_char_p, C.c_char_p, pvp]),
    "cacti_tensors_dir_close": (ci, [vp]),
    "cacti_tensors_dir_count": (ci, [vp]),
    "cacti_tensors_dir_entry": (ci, [vp, ci, C.c_char_p, sz, C.c_char_p, sz, C.POINTER(ci), C.POINTER(i64), pvp,
                                C.POINTER(C.c_uint64)]),
    "cacti_cell_matcher_match": (ci, [vp, ci, vp, ci, vp]),
    "cacti_llama_load_tensors_dir": (ci, [vp, vp, C.POINTER(ci)]),
    "cacti_llama_cached_create": (ci, [vp, i64, pvp]),
    "cacti_llama_cached_destroy": (ci, [vp]),
    "cacti_llama_cached_reset_state": (ci, [vp]),
    "cacti_llama_cached_set_tokens": (ci, [vp, vp, i64]),
    "cacti_llama_cached_get_tokens": (ci, [vp, vp]),
    "cacti_llama_cached_apply": (ci, [vp, i64, i64, ci]),
    "cacti_llama_cached_outputs": (ci, [vp, vp, vp, vp]),
    "cacti_llama_adamw_init": (ci, [vp]),
    "cacti_llama_adamw_step": (ci, [vp, ci, vp, ci]),
    "cacti_llama_adamw_state_get": (ci, [vp, ci, ci, vp, sz]),
    "cacti_llama_io_cells": (ci, [vp] + [C.POINTER(ci)] * 7),
    "cacti_llama_set_attention": (ci, [vp, ci]),
    "cacti_llama_set_product_groups": (ci, [vp, ci]),
    "cacti_llama_stage": (ci, [vp, ci, ci]),
    "cacti_llama_step": (ci, [vp, vp, vp, vp, ci, ci, vp]),
}


class AdamW32(C.Structure):
    """cacti_adamw32 (AdamW32, src/librarium/adamw.rs:4-28)."""
    _fields_ = [("grad_scale", f32), ("lr", f32), ("wd", f32), ("a1", f32), ("a2", f32), ("eps", f32)]


class LlamaCfg(C.Structure):
    _fields_ = [("S", i64), ("D", i64), ("H", i64), ("Dh", i64), ("F", i64), ("V", i64),
                ("L", i64), ("eps", f32)]


class Stats(C.Structure):
    _fields_ = [(n, C.c_uint64) for n in (
        "pool_cap", "pool_used", "pool_peak", "pool_front", "n_alloc", "n_evict", "n_upload",
        "bytes_d2h", "bytes_h2d", "n_soft_oom", "n_entries", "n_thunks_run", "host_bytes")]

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
