"""The driver-level entry points of the C ABI on a device (MI355X): memory, streams, events, the primary
context and the null stream (cacti_gpu_cu_ffi/src/lib.rs:98-565), and the device reserve sized from the
environment (src/pctx/nvgpu.rs:1434-1463)."""
import ctypes as C
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def test_memory_streams_events_round_trip():
    from cacti_amd import ffi
    n = C.c_int()
    ffi.call("cacti_hip_device_count", C.byref(n))
    assert n.value >= 1
    ffi.call("cacti_hip_device_set", 0)
    free_b, total_b = C.c_size_t(), C.c_size_t()
    ffi.call("cacti_hip_mem_get_info", C.byref(free_b), C.byref(total_b))
    assert 0 < free_b.value <= total_b.value
    nbytes = 1 << 20
    dptr, hsrc, hdst, st, e0, e1 = (C.c_void_p() for _ in range(6))
    ffi.call("cacti_hip_mem_alloc", C.byref(dptr), nbytes)
    ffi.call("cacti_hip_mem_alloc_host", C.byref(hsrc), nbytes)
    ffi.call("cacti_hip_mem_alloc_host", C.byref(hdst), nbytes)
    src = np.ctypeslib.as_array(C.cast(hsrc, C.POINTER(C.c_uint8)), (nbytes,))
    dst = np.ctypeslib.as_array(C.cast(hdst, C.POINTER(C.c_uint8)), (nbytes,))
    src[:] = np.random.default_rng(0).integers(0, 256, nbytes, dtype=np.uint8)
    dst[:] = 0
    ffi.call("cacti_hip_stream_create_nonblocking", C.byref(st))
    ffi.call("cacti_hip_event_create", C.byref(e0), 1)
    ffi.call("cacti_hip_event_create", C.byref(e1), 1)
    ffi.call("cacti_hip_event_record", e0, st)
    ffi.call("cacti_hip_memcpy_h2d_async", dptr, hsrc, nbytes, st)
    ffi.call("cacti_hip_memcpy_d2h_async", hdst, dptr, nbytes, st)
    ffi.call("cacti_hip_event_record", e1, st)
    ffi.call("cacti_hip_event_sync", e1)
    ms = C.c_float()
    ffi.call("cacti_hip_event_elapsed_ms", e0, e1, C.byref(ms))
    assert ms.value > 0 and np.array_equal(src, dst)
    # the same through the null stream's handle
    null = ffi.lib().cacti_hip_stream_null()
    assert null is None
    dst[:] = 0
    ffi.call("cacti_hip_memset_async", dptr, 0x5A, nbytes, null)
    ffi.call("cacti_hip_memcpy_d2h_async", hdst, dptr, nbytes, null)
    ffi.call("cacti_hip_stream_sync", null)
    assert np.all(dst == 0x5A)
    for ev in (e0, e1):
        ffi.call("cacti_hip_event_destroy", ev)
    ffi.call("cacti_hip_stream_destroy", st)
    ffi.call("cacti_hip_mem_free", dptr)
    ffi.call("cacti_hip_mem_free_host", hsrc)
    ffi.call("cacti_hip_mem_free_host", hdst)


def test_primary_context_retain_release():
    from cacti_amd import ffi
    a, b = C.c_void_p(), C.c_void_p()
    ffi.call("cacti_hip_primary_ctx_retain", 0, C.byref(a))
    ffi.call("cacti_hip_primary_ctx_retain", 0, C.byref(b))
    assert a.value is not None and a.value == b.value          # one primary context per device
    ffi.call("cacti_hip_primary_ctx_release", 0)
    ffi.call("cacti_hip_primary_ctx_release", 0)
    with pytest.raises(ffi.CactiError):
        ffi.call("cacti_hip_primary_ctx_retain", 4096, C.byref(a))   # no such device: a status, not an abort
    # flags of a primary context that is already active (torch made it so): a status, not an abort
    try:
        ffi.call("cacti_hip_primary_ctx_set_flags", 0, 0)
    except ffi.CactiError as e:
        assert e.code > 0                                       # the runtime's hipError_t
    # a reset is refused while a device context of this library lives on the device (nothing is reset here)
    from cacti_amd.runtime import Ctx
    ctx = Ctx(0, 64 << 20, 0)
    with pytest.raises(ffi.CactiError) as e:
        ffi.call("cacti_hip_primary_ctx_reset", 0)
    assert e.value.code == -5 and "alive" in str(e.value)
    ctx.close()
    # a reported failure does not linger as the status of the next kernel launch
    import torch
    from cacti_amd import ops
    x = torch.ones(8, 16, device="cuda", dtype=torch.float16)
    assert torch.equal(ops.add_f16(x, x), x + x)


def test_reserve_sized_from_the_environment(monkeypatch):
    from cacti_amd.runtime import Ctx
    monkeypatch.setenv("CACTI_VMEM_SOFT_LIMIT", "1GiB")
    monkeypatch.setenv("CACTI_GPU_MEM_ALLOC", "pagelocked")
    ctx = Ctx(0, 0, -1)
    assert ctx.stats()["pool_cap"] == 1 << 30
    ctx.close()
    monkeypatch.setenv("CACTI_VMEM_SOFT_LIMIT", "0.01")
    ctx = Ctx(0, 0, -1)
    from cacti_amd import ffi
    free_b, total_b = C.c_size_t(), C.c_size_t()
    ffi.call("cacti_hip_mem_get_info", C.byref(free_b), C.byref(total_b))
    assert ctx.stats()["pool_cap"] == int(total_b.value * 0.01) >> 16 << 16
    ctx.close()
    monkeypatch.setenv("CACTI_VMEM_SOFT_LIMIT", "100000GiB")
    with pytest.raises(ffi.CactiError) as e:
        Ctx(0, 0, -1)
    assert e.value.code == -4 and "CACTI_VMEM_SOFT_LIMIT" in str(e.value)
    monkeypatch.setenv("CACTI_VMEM_SOFT_LIMIT", "2GiB")
    ctx = Ctx(0, 256 << 20, 0)                                  # an explicit cap wins over the environment
    assert ctx.stats()["pool_cap"] == 256 << 20
    ctx.close()
