"""Operator-level Python mirror of the thunks on cacti's LLaMA backward path.

Each function is one `ThunkImpl::apply` (or `accumulate` when an `*_acc` tensor is
given) in the reference's terms (src/thunk/mod.rs:347-351), executed by the HIP kernels
behind the C ABI.  torch is used only to own device memory and name the stream; every
computation goes through libcacti_gpu_hip_ffi.so and fails if it is not built.
"""
import torch

from . import ffi

F16 = torch.float16


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _p(t):
    return 0 if t is None else t.data_ptr()


def _chk(t, dtype=F16):
    assert t.is_cuda and t.is_contiguous() and t.dtype == dtype, (t.dtype, t.device, t.shape)
    return t


def selftest_wave_reduce():
    out = torch.zeros(4, dtype=torch.float32, device="cuda")
    ffi.call("cacti_hip_selftest_wave_reduce", out.data_ptr(), _stream())
    return out.cpu().tolist()


# ---------------------------------------------------------------- GEMM
def gemm(a, b, ta=False, tb=False, alpha=1.0, beta=0.0, out=None):
    """out = f16(alpha op(a) op(b) + beta out); a, b 2-d row-major f16 (rows may be strided)."""
    assert a.dim() == 2 and b.dim() == 2 and a.stride(1) == 1 and b.stride(1) == 1
    M, K = (a.shape[1], a.shape[0]) if ta else a.shape
    K2, N = (b.shape[1], b.shape[0]) if tb else b.shape
    assert K == K2, (a.shape, b.shape, ta, tb)
    if out is None:
        assert beta == 0.0
        out = torch.empty((M, N), dtype=F16, device=a.device)
    assert out.shape == (M, N) and out.stride(1) == 1
    ffi.call("cacti_hip_gemm_f16", int(ta), int(tb), M, N, K, alpha, a.data_ptr(), a.stride(0),
             b.data_ptr(), b.stride(0), beta, out.data_ptr(), out.stride(0), _stream())
    return out


def gemm_batched(As, Bs, ta=False, tb=False, alpha=1.0, beta=0.0, outs=None):
    """Pointer-array batch: outs[z] = f16(alpha op(As[z]) op(Bs[z]) + beta outs[z]), one shape."""
    import ctypes as C
    n = len(As)
    a, b = As[0], Bs[0]
    M, K = (a.shape[1], a.shape[0]) if ta else a.shape
    N = b.shape[0] if tb else b.shape[1]
    if outs is None:
        assert beta == 0.0
        outs = [torch.empty((M, N), dtype=F16, device=a.device) for _ in range(n)]
    arr = lambda ts: C.cast((C.c_void_p * n)(*[t.data_ptr() for t in ts]), C.c_void_p)
    ffi.call("cacti_hip_gemm_f16_batched", int(ta), int(tb), n, M, N, K, alpha, arr(As), a.stride(0), arr(Bs),
             b.stride(0), beta, arr(outs), outs[0].stride(0), _stream())
    return outs


def gemm_strided_batched(ta, tb, nblk, M, N, K, alpha, a, lda, sa, b, ldb, sb, beta, c, ldc, sc,
                         tri=0):
    """tri: 0 dense; 1 only tril(C) wanted (rest unwritten); 2 A = tril; 3 A^T with A = tril."""
    ffi.call("cacti_hip_gemm_f16_strided_batched_tri", int(ta), int(tb), nblk, M, N, K, alpha,
             a.data_ptr(), lda, sa, b.data_ptr(), ldb, sb, beta, c.data_ptr(), ldc, sc, int(tri),
             _stream())
    return c


def block_matmul_qk(q, k, alpha, causal=False):
    """S16[i,h,j] = f16(alpha q[i,h,:] . k[j,h,:]) on [S,H,Dh] tensors (src/librarium/llama.rs:501).
    causal: only the tiles touching j <= i are computed; the rest of S16 is left unwritten."""
    S, H, Dh = q.shape
    s16 = torch.empty((S, H, S), dtype=F16, device=q.device)
    return gemm_strided_batched(False, True, H, S, S, Dh, alpha, q, H * Dh, Dh, k, H * Dh, Dh, 0.0,
                                s16, H * S, S, tri=1 if causal else 0)


def block_matmul_pv(p16, v, causal=False):
    """O[i,h,:] = f16(sum_j p16[i,h,j] v[j,h,:]) (src/librarium/llama.rs:506).
    causal: p16 is lower triangular (as the causal softmax writes it)."""
    S, H, _ = p16.shape
    Dh = v.shape[2]
    o = torch.empty((S, H, Dh), dtype=F16, device=v.device)
    return gemm_strided_batched(False, False, H, S, Dh, S, 1.0, p16, H * S, S, v, H * Dh, Dh, 0.0, o,
                                H * Dh, Dh, tri=2 if causal else 0)


def attention_fwd(q, k, v, alpha):
    """Fused causal attention on [S,H,Dh] tensors: returns (o, stats); stats feeds attention_bwd."""
    _chk(q), _chk(k), _chk(v)
    S, H, Dh = q.shape
    o = torch.empty_like(q)
    stats = torch.empty(ffi.lib().cacti_hip_attention_stats_bytes(S, H) // 4, dtype=torch.float32, device=q.device)
    ffi.call("cacti_hip_attention_fwd", S, H, Dh, alpha, q.data_ptr(), k.data_ptr(), v.data_ptr(), H * Dh,
             o.data_ptr(), stats.data_ptr(), _stream())
    return o, stats


def attention_bwd(q, k, v, dO, stats, alpha, acc=None, o=None):
    """Adjoint of attention_fwd: returns (dq, dk, dv); acc = (dq, dk, dv) to accumulate into; o = the forward
    output (lets blocks of queries with spread probabilities skip the pass that forms the row sums)."""
    _chk(q), _chk(k), _chk(v), _chk(dO)
    if o is not None:
        _chk(o)
    S, H, Dh = q.shape
    dq, dk, dv = acc if acc is not None else (torch.empty_like(q), torch.empty_like(q), torch.empty_like(q))
    a = int(acc is not None)
    nbytes = ffi.lib().cacti_hip_attention_bwd_workspace(S, H)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=q.device)
    ffi.call("cacti_hip_attention_bwd", S, H, Dh, alpha, q.data_ptr(), k.data_ptr(), v.data_ptr(),
             0 if o is None else o.data_ptr(), dO.data_ptr(), H * Dh, stats.data_ptr(), dq.data_ptr(), a,
             dk.data_ptr(), a, dv.data_ptr(), a,
             ws.data_ptr(), nbytes, _stream())
    return dq, dk, dv


# ---------------------------------------------------------------- fused thunks
def rms_norm_fwd(x, w, eps):
    _chk(x), _chk(w)
    N, D = x.shape
    y = torch.empty_like(x)
    ffi.call("cacti_hip_rms_norm_fwd", N, D, x.data_ptr(), w.data_ptr(), eps, y.data_ptr(),
             _stream())
    return y


def add_rms_norm_fwd(a, b, w, eps):
    """(f16(a + b), rms_norm of it): the residual add and the norm that follows, one launch."""
    _chk(a), _chk(b), _chk(w)
    N, D = a.shape
    s, y = torch.empty_like(a), torch.empty_like(a)
    ffi.call("cacti_hip_add_rms_norm_fwd", N, D, a.data_ptr(), b.data_ptr(), w.data_ptr(), eps,
             s.data_ptr(), y.data_ptr(), _stream())
    return s, y


def rms_norm_bwd(x, w, eps, dy, dx_acc=None, dw_acc=None):
    """Returns (dx, dw).  dx_acc / dw_acc: tensors to accumulate into (updated in place)."""
    _chk(x), _chk(w), _chk(dy)
    N, D = x.shape
    dx = torch.empty_like(x) if dx_acc is None else _chk(dx_acc)
    dw = torch.empty_like(w) if dw_acc is None else _chk(dw_acc)
    nbytes = ffi.lib().cacti_hip_rms_norm_bwd_workspace(N, D)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=x.device)
    ffi.call("cacti_hip_rms_norm_bwd", N, D, x.data_ptr(), w.data_ptr(), eps, dy.data_ptr(),
             dx.data_ptr(), int(dx_acc is not None), dw.data_ptr(), int(dw_acc is not None),
             ws.data_ptr(), nbytes, _stream())
    return dx, dw


def rope_tables(S, Dh, device="cuda"):
    cos = torch.empty((S, Dh), dtype=F16, device=device)
    sin = torch.empty((S, Dh), dtype=F16, device=device)
    ffi.call("cacti_hip_rope_tables", S, Dh, cos.data_ptr(), sin.data_ptr(), _stream())
    return cos, sin


def rope_fwd(x, cos, sin):
    _chk(x), _chk(cos), _chk(sin)
    S, H, Dh = x.shape
    y = torch.empty_like(x)
    ffi.call("cacti_hip_rope_fwd", S, H, Dh, x.data_ptr(), cos.data_ptr(), sin.data_ptr(),
             y.data_ptr(), _stream())
    return y


def rope_bwd(dy, cos, sin, dx_acc=None):
    _chk(dy), _chk(cos), _chk(sin)
    S, H, Dh = dy.shape
    dx = torch.empty_like(dy) if dx_acc is None else _chk(dx_acc)
    ffi.call("cacti_hip_rope_bwd", S, H, Dh, dy.data_ptr(), cos.data_ptr(), sin.data_ptr(),
             dx.data_ptr(), int(dx_acc is not None), _stream())
    return dx


def silu_gate_fwd(g, u):
    _chk(g), _chk(u)
    h = torch.empty_like(g)
    ffi.call("cacti_hip_silu_gate_fwd", g.numel(), g.data_ptr(), u.data_ptr(), h.data_ptr(),
             _stream())
    return h


def silu_gate_bwd(g, u, dh, dg_acc=None, du_acc=None):
    _chk(g), _chk(u), _chk(dh)
    dg = torch.empty_like(g) if dg_acc is None else _chk(dg_acc)
    du = torch.empty_like(g) if du_acc is None else _chk(du_acc)
    ffi.call("cacti_hip_silu_gate_bwd", g.numel(), g.data_ptr(), u.data_ptr(), dh.data_ptr(),
             dg.data_ptr(), int(dg_acc is not None), du.data_ptr(), int(du_acc is not None),
             _stream())
    return dg, du


def causal_softmax_fwd(s16):
    _chk(s16)
    S, H, S2 = s16.shape
    assert S == S2
    # the kernel writes j <= i and zeros only up to the next multiple of 256 columns:
    # start from zeros so that dense consumers may read the whole row
    p = torch.zeros_like(s16)
    ffi.call("cacti_hip_causal_softmax_fwd", S, H, s16.data_ptr(), p.data_ptr(), _stream())
    return p


def causal_softmax_bwd(s16, dp16):
    _chk(s16), _chk(dp16)
    S, H, _ = s16.shape
    ds = torch.zeros_like(s16)
    ffi.call("cacti_hip_causal_softmax_bwd", S, H, s16.data_ptr(), dp16.data_ptr(), ds.data_ptr(),
             _stream())
    return ds


def _raise_index(status, what):
    v = int(status.item())
    if v:
        raise IndexError("%s: id out of range at row %d" % (what, v - 1))


def softmax_ce_fwd(logit, tok, want_prob=True):
    """Returns (prob f32 or None, loss f32 [N], amax u16-as-int16 bits [N])."""
    _chk(logit)
    N, V = logit.shape
    prob = torch.empty((N, V), dtype=torch.float32, device=logit.device) if want_prob else None
    loss = torch.empty((N,), dtype=torch.float32, device=logit.device)
    amax = torch.empty((N,), dtype=torch.int16, device=logit.device)
    status = torch.zeros(1, dtype=torch.int32, device=logit.device)
    ffi.call("cacti_hip_softmax_ce_fwd", N, V, logit.data_ptr(), tok.data_ptr(), _p(prob),
             loss.data_ptr(), amax.data_ptr(), status.data_ptr(), _stream())
    _raise_index(status, "softmax_ce_fwd")
    return prob, loss, amax


def softmax_ce_bwd(logit, tok, scale, acc=None):
    _chk(logit), _chk(scale, torch.float32)
    N, V = logit.shape
    d = torch.empty_like(logit) if acc is None else _chk(acc)
    ffi.call("cacti_hip_softmax_ce_bwd", N, V, logit.data_ptr(), tok.data_ptr(), scale.data_ptr(),
             d.data_ptr(), int(acc is not None), _stream())
    return d


def embed_fwd(W, tok):
    _chk(W)
    V, D = W.shape
    S = tok.numel()
    y = torch.empty((S, D), dtype=F16, device=W.device)
    status = torch.zeros(1, dtype=torch.int32, device=W.device)
    ffi.call("cacti_hip_embed_fwd", V, D, W.data_ptr(), S, tok.data_ptr(), y.data_ptr(),
             status.data_ptr(), _stream())
    _raise_index(status, "embed_fwd")
    return y


def embed_bwd(V, tok, dy, acc=None):
    _chk(dy)
    S, D = dy.shape
    dW = torch.empty((V, D), dtype=F16, device=dy.device) if acc is None else _chk(acc)
    ffi.call("cacti_hip_embed_bwd", V, D, S, tok.data_ptr(), dy.data_ptr(), dW.data_ptr(),
             int(acc is not None), _stream())
    return dW


def add_f16(a, b, out=None):
    out = torch.empty_like(a) if out is None else out
    ffi.call("cacti_hip_add_f16", a.numel(), a.data_ptr(), b.data_ptr(), out.data_ptr(), _stream())
    return out


def accumulate_1d(dst, src):
    name = {torch.float32: "f32", torch.float16: "f16", torch.int16: "u16"}[dst.dtype]
    ffi.call("cacti_hip_accumulate_1d_" + name, dst.data_ptr(), src.data_ptr(), dst.numel(),
             _stream())
    return dst


# ---------------------------------------------------------------- numerical-health digests
def nan_count(x):
    """Number of NaNs of an f16 tensor as a 0-d int64 device tensor (src/thunk/op.rs:273-349)."""
    _chk(x)
    out = torch.empty((), dtype=torch.int64, device=x.device)
    ffi.call("cacti_hip_nan_count_f16", x.numel(), x.data_ptr(), out.data_ptr(), _stream())
    return out


def abs_log2_hist8(x):
    """int64[256] histogram of the floor(log2 |x|) classes of an f16 tensor (src/thunk/op.rs:351-441)."""
    _chk(x)
    out = torch.empty(256, dtype=torch.int64, device=x.device)
    ffi.call("cacti_hip_abs_log2_hist8_f16", x.numel(), x.data_ptr(), out.data_ptr(), _stream())
    return out


def digests(xs):
    """Both digests of a list of f16 tensors in one launch: (hist int64[n,256], nan int64[n])
    (the per-cycle loop of examples/open_llama_3b_train.rs:409-424)."""
    import ctypes as C
    n = len(xs)
    for x in xs:
        _chk(x)
    dev = xs[0].device if n else torch.device("cuda")
    out = torch.empty((n, 257), dtype=torch.int64, device=dev)
    if n == 0:
        return out[:, :256], out[:, 256]
    scratch = torch.empty(ffi.lib().cacti_hip_digests_scratch_bytes(n), dtype=torch.uint8, device=dev)
    ptrs = (C.c_void_p * n)(*[x.data_ptr() for x in xs])
    ns = (C.c_int64 * n)(*[x.numel() for x in xs])
    ffi.call("cacti_hip_digests_f16_batch", n, C.cast(ptrs, C.c_void_p), C.cast(ns, C.c_void_p),
             out.data_ptr(), scratch.data_ptr(), _stream())
    return out[:, :256], out[:, 256]


# ---------------------------------------------------------------- optimiser thunks (AdamW32)
def _f(x):
    return _chk(x, torch.float32)


def online_average_scale_(u, v, src_scale, rate):
    """v += rate * (src_scale * f32(u) - v) in place (src/thunk/op.rs:3884-3939)."""
    _chk(u), _f(v)
    assert u.numel() == v.numel()
    ffi.call("cacti_hip_online_average_scale_f16_f32", u.numel(), u.data_ptr(), v.data_ptr(), src_scale, rate,
             _stream())
    return v


def online_average_square_scale_(u, v, src_scale, rate):
    """v += rate * ((src_scale * f32(u))^2 - v) in place (src/thunk/op.rs:3941-4002)."""
    _chk(u), _f(v)
    assert u.numel() == v.numel()
    ffi.call("cacti_hip_online_average_square_scale_f16_f32", u.numel(), u.data_ptr(), v.data_ptr(), src_scale,
             rate, _stream())
    return v


def online_adamw_update_(g1, g2, w, signed_lr, lr_unbias, lamda, eps):
    """w += signed_lr * (lr_unbias * (g1 / (sqrt(g2) + eps)) + lamda * w) in place
    (src/thunk/op.rs:4004-4062)."""
    _f(g1), _f(g2), _f(w)
    assert g1.numel() == g2.numel() == w.numel()
    ffi.call("cacti_hip_online_adamw_update_f32", w.numel(), g1.data_ptr(), g2.data_ptr(), w.data_ptr(),
             signed_lr, lr_unbias, lamda, eps, _stream())
    return w


def cast_f32_f16(x):
    _f(x)
    y = torch.empty(x.shape, dtype=torch.float16, device=x.device)
    ffi.call("cacti_hip_cast_f32_f16", x.numel(), x.data_ptr(), y.data_ptr(), _stream())
    return y


def cast_f16_f32(x):
    _chk(x)
    y = torch.empty(x.shape, dtype=torch.float32, device=x.device)
    ffi.call("cacti_hip_cast_f16_f32", x.numel(), x.data_ptr(), y.data_ptr(), _stream())
    return y


def adamw32_scalars(iter_nr, grad_scale, lr, wd, a1, a2, eps):
    """The seven f32 scalars of one AdamW32 step (host arithmetic of src/librarium/adamw.rs:45-60 and
    src/op.rs:984-1023) as a list; raises for iter_nr <= 0."""
    import ctypes as C
    out = (C.c_float * 7)()
    ffi.call("cacti_adamw32_scalars", int(iter_nr), grad_scale or 0.0, lr, wd, a1, a2, eps, C.cast(out, C.c_void_p))
    return list(out)


def adamw32_step_(grads, avgs, avg2s, masters, params, scalars):
    """One AdamW32 step of a list of tensors in one launch, in place (avgs, avg2s, masters updated,
    params overwritten with f16(master))."""
    import ctypes as C
    n = len(grads)
    assert len(avgs) == len(avg2s) == len(masters) == len(params) == n
    if n == 0:
        return
    for g, a, b, w, p in zip(grads, avgs, avg2s, masters, params):
        _chk(g), _f(a), _f(b), _f(w), _chk(p)
        assert g.numel() == a.numel() == b.numel() == w.numel() == p.numel()
    arr = lambda ts: C.cast((C.c_void_p * n)(*[t.data_ptr() for t in ts]), C.c_void_p)
    ns = (C.c_int64 * n)(*[g.numel() for g in grads])
    sc = (C.c_float * 7)(*scalars)
    scratch = torch.empty(ffi.lib().cacti_hip_adamw32_scratch_bytes(n), dtype=torch.uint8, device=grads[0].device)
    ffi.call("cacti_hip_adamw32_step_f16_batch", n, arr(grads), arr(avgs), arr(avg2s), arr(masters), arr(params),
             C.cast(ns, C.c_void_p), C.cast(sc, C.c_void_p), scratch.data_ptr(), _stream())


# ---------------------------------------------------------------- bf16 raw casts (src/thunk/op.rs:665-803)
def _raw_cast(name, x, in_dtype, out_dtype):
    _chk(x, in_dtype)
    y = torch.empty(x.shape, dtype=out_dtype, device=x.device)
    ffi.call(name, x.numel(), x.data_ptr(), y.data_ptr(), _stream())
    return y


def raw_cast_bf16_f16(u):
    """bf16 bit patterns (int16 tensor) -> f16."""
    return _raw_cast("cacti_hip_raw_cast_bf16_f16", u, torch.int16, torch.float16)


def raw_cast_bf16_f32(u):
    return _raw_cast("cacti_hip_raw_cast_bf16_f32", u, torch.int16, torch.float32)


def raw_cast_f32_bf16(x):
    """f32 -> bf16 bit patterns (int16 tensor), truncating."""
    return _raw_cast("cacti_hip_raw_cast_f32_bf16", x, torch.float32, torch.int16)


def raw_cast_f16_bf16(x):
    return _raw_cast("cacti_hip_raw_cast_f16_bf16", x, torch.float16, torch.int16)
