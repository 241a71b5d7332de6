"""The adjoint entry point that allocates nothing (`cacti_hip_rms_norm_bwd_static`): same bits as
`cacti_hip_rms_norm_bwd` with a caller workspace, on two calls in a row, the second smaller, so that
what the first call left in the built-in buffer is there when the second one runs."""
import ctypes

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

EPS = 1e-6


def _both(torch, ffi, N, D, seed, acc):
    r = np.random.default_rng(seed)
    dev = lambda a: torch.from_numpy(a).cuda()
    x, dy = (dev(r.standard_normal((N, D)).astype(np.float16)) for _ in range(2))
    w = dev(r.standard_normal(D).astype(np.float16))
    dx0 = dev(r.standard_normal((N, D)).astype(np.float16))
    dw0 = dev(r.standard_normal(D).astype(np.float16))
    st = torch.cuda.current_stream().cuda_stream
    outs = []
    for static in (False, True):
        dx, dw = dx0.clone(), dw0.clone()
        torch.cuda.synchronize()
        before = torch.cuda.memory_allocated()
        free0, tot = ctypes.c_size_t(), ctypes.c_size_t()
        ffi.call("cacti_hip_mem_get_info", ctypes.byref(free0), ctypes.byref(tot))
        if static:
            ffi.call("cacti_hip_rms_norm_bwd_static", N, D, x.data_ptr(), w.data_ptr(), EPS, dy.data_ptr(),
                     dx.data_ptr(), acc, dw.data_ptr(), acc, st)
            torch.cuda.synchronize()
            free1 = ctypes.c_size_t()
            ffi.call("cacti_hip_mem_get_info", ctypes.byref(free1), ctypes.byref(tot))
            assert torch.cuda.memory_allocated() == before and free1.value == free0.value
        else:
            nbytes = ffi.lib().cacti_hip_rms_norm_bwd_workspace(N, D)
            ws = torch.full((nbytes,), 0xFF, dtype=torch.uint8, device="cuda")
            ffi.call("cacti_hip_rms_norm_bwd", N, D, x.data_ptr(), w.data_ptr(), EPS, dy.data_ptr(),
                     dx.data_ptr(), acc, dw.data_ptr(), acc, ws.data_ptr(), nbytes, st)
        torch.cuda.synchronize()
        outs.append((dx.cpu().numpy().view(np.uint16), dw.cpu().numpy().view(np.uint16)))
    return outs


def test_static_scratch_adjoint_matches_the_workspace_one_twice_in_a_row():
    import torch
    from cacti_amd import ffi
    print("case: rms_norm_bwd_static [2048,3200] acc=1 then [72,256] acc=0", flush=True)
    for (N, D, seed, acc) in ((2048, 3200, 11, 1), (72, 256, 12, 0)):
        (dx_a, dw_a), (dx_b, dw_b) = _both(torch, ffi, N, D, seed, acc)
        assert np.array_equal(dx_a, dx_b), "dx differs at N=%d D=%d" % (N, D)
        assert np.array_equal(dw_a, dw_b), "dw differs at N=%d D=%d" % (N, D)


def test_static_scratch_adjoint_rejects_what_does_not_fit():
    from cacti_amd import ffi
    L = ffi.lib()
    cap = L.cacti_hip_rms_norm_bwd_static_max_bytes()
    assert cap == 8 << 20
    N, D = 8 * 300, 8192                      # 300 partial rows of 32 KiB = 9.4 MiB
    assert L.cacti_hip_rms_norm_bwd_workspace(N, D) > cap
    rc = L.cacti_hip_rms_norm_bwd_static(N, D, 256, 256, ctypes.c_float(EPS), 256, 256, 0, 256, 0, None)
    assert rc == -1 and b"scratch" in L.cacti_hip_last_error()
