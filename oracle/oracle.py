"""ctypes binding of the CPU oracle (oracle/cacti_oracle.c).

TEST INFRASTRUCTURE.  Only tests/, __graft_entry__.smoke() and the cpu_baseline
leg of bench.py may import this module; the product never does.

Arrays are numpy: f16 tensors as np.float16 (or uint16 views), indices uint16.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None

i64 = C.c_int64
f32 = C.c_float
vp = C.c_void_p


def build(force=False):
    """Compile both oracle variants with gcc via the Makefile."""
    if force:
        subprocess.check_call(["make", "-C", _HERE, "clean"], stdout=subprocess.DEVNULL)
    subprocess.check_call(["make", "-C", _HERE, "-j2"], stdout=subprocess.DEVNULL)


def _cpu_has_avx2():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("flags"):
                    fl = set(line.split(":", 1)[1].split())
                    return {"avx2", "fma"} <= fl
    except OSError:
        pass
    return False


def lib():
    global _LIB
    if _LIB is None:
        name = "liboracle_avx2.so" if _cpu_has_avx2() else "liboracle_generic.so"
        path = os.path.join(_HERE, name)
        if not os.path.exists(path):
            build()
        _LIB = C.CDLL(path)
        _LIB.oracle_h2f.restype = f32
        _LIB.oracle_h2f.argtypes = [C.c_uint16]
        _LIB.oracle_f2h.restype = C.c_uint16
        _LIB.oracle_f2h.argtypes = [f32]
        _LIB.oracle_llama_step.restype = i64
        _LIB.oracle_softmax_ce_fwd.restype = i64
        _LIB.oracle_softmax_ce_bwd.restype = i64
        _LIB.th_softmax_nll_f32.restype = i64
        _LIB.th_outer_select_f16.restype = i64
        _LIB.oracle_layer_elems.restype = i64
        _LIB.oracle_nan_count_f16.restype = i64
        _LIB.oracle_abs_log2_bin.restype = C.c_int
        _LIB.oracle_abs_log2_bin.argtypes = [C.c_uint16]
        _LIB.oracle_param_elems.restype = i64
        _LIB.oracle_num_threads.restype = C.c_int
    return _LIB


def P(a):
    """Pointer to a C-contiguous numpy array (or None)."""
    if a is None:
        return vp(0)
    assert a.flags["C_CONTIGUOUS"], "oracle arrays must be contiguous"
    return vp(a.ctypes.data)


def h(a):
    """np.float16 array from anything."""
    return np.ascontiguousarray(np.asarray(a, dtype=np.float16))


class Cfg(C.Structure):
    _fields_ = [("S", i64), ("D", i64), ("H", i64), ("Dh", i64), ("F", i64), ("V", i64),
                ("L", i64), ("eps", f32)]


def num_threads():
    return lib().oracle_num_threads()


def set_gemm_reverse_k(on):
    """Sum GEMM products in descending k (an equally valid fp32 accumulation order)."""
    lib().oracle_set_gemm_reverse_k(C.c_int(int(on)))


# fp32 summation orders of the oracle's GEMMs as (run, rev, tree): k cut into runs of `run` values
# (0 = one run), each summed ascending (rev: descending) from zero; run sums added in order or as a tree
GEMM_ORDERS = {"ascending": (0, 0, 0), "descending": (0, 1, 0), "blocked64": (64, 0, 0), "pairwise": (32, 0, 1),
               "blocked16": (16, 0, 0), "blocked64rev": (64, 1, 0), "pairwise8": (8, 0, 1), "blocked256": (256, 0, 0)}


def set_gemm_order(mode):
    """fp32 summation order of every oracle GEMM: a key of GEMM_ORDERS or a (run, rev, tree) tuple."""
    run, rev, tree = GEMM_ORDERS.get(mode, mode)
    lib().oracle_set_gemm_order_ex(C.c_int(run), C.c_int(rev), C.c_int(tree))


def set_norm_reciprocal(on):
    """RMSNorm divides (0, the reference's lambda) or multiplies by the reciprocal (1, <= 1 fp32 ulp away)."""
    lib().oracle_set_norm_reciprocal(C.c_int(int(on)))


def set_reduce_f32(on):
    """Row / column reductions accumulate in f32, ascending (1), instead of f64 then one rounding (0)."""
    lib().oracle_set_reduce_f32(C.c_int(int(on)))


def set_exp_exact(on):
    """exp / log correctly rounded through double (1) instead of libm's expf / logf (0)."""
    lib().oracle_set_exp_exact(C.c_int(int(on)))


# Restatements of the cycle that differ only in what the reference leaves open: the fp32 summation
# order of its GEMMs (cuBLAS), the association order of its f32 reductions (Futhark) and the last ulp
# of exp / log (libm).  (gemm order, reduce_f32, exp_exact); the first one is the default oracle.
RESTATEMENTS = {
    "ascending": ("ascending", 0, 0),
    "descending": ("descending", 0, 0),
    "blocked64": ("blocked64", 0, 0),
    "pairwise": ("pairwise", 0, 0),
    "ascending+f32sums": ("ascending", 1, 0),
    "blocked64+f32sums+exp": ("blocked64", 1, 1),
    "pairwise+exp": ("pairwise", 0, 1),
    "descending+f32sums+exp": ("descending", 1, 1),
    "blocked16": ("blocked16", 0, 0),
    "blocked64rev+f32sums": ("blocked64rev", 1, 0),
    "pairwise8+exp": ("pairwise8", 0, 1),
    "blocked256+f32sums+exp": ("blocked256", 1, 1),
}


def set_restatement(name):
    order, red, ex = RESTATEMENTS[name]
    set_gemm_order(order)
    set_reduce_f32(red)
    set_exp_exact(ex)


def set_num_threads(n):
    lib().oracle_set_num_threads(C.c_int(n))


# --------------------------------------------------------------------------
# fused units

def rope_tables(S, Dh):
    cos = np.empty((S, Dh), np.float16)
    sin = np.empty((S, Dh), np.float16)
    lib().oracle_rope_tables(i64(S), i64(Dh), P(cos), P(sin))
    return cos, sin


def rmsnorm_fwd(x, w, eps):
    N, D = x.shape
    y = np.empty((N, D), np.float16)
    t = np.empty((N, D), np.float32)
    s = np.empty((N,), np.float32)
    lib().oracle_rmsnorm_fwd(i64(N), i64(D), P(x), P(w), f32(eps), P(y), P(t), P(s))
    return y, t, s


def rmsnorm_bwd(x, w, eps, dy, dx_init=None, dw_init=None):
    """Returns (dx, dw); *_init given => Accumulate into a copy of it."""
    N, D = x.shape
    _, t, s = rmsnorm_fwd(x, w, eps)
    dx = np.empty((N, D), np.float16) if dx_init is None else dx_init.copy()
    dw = np.empty((D,), np.float16) if dw_init is None else dw_init.copy()
    lib().oracle_rmsnorm_bwd(i64(N), i64(D), P(x), P(w), P(t), P(s), P(dy), P(dx),
                             C.c_int(dx_init is not None), P(dw), C.c_int(dw_init is not None))
    return dx, dw


def rope_fwd(x, cos, sin):
    S, H, Dh = x.shape
    y = np.empty_like(x)
    lib().oracle_rope_fwd(i64(S), i64(H), i64(Dh), P(x), P(cos), P(sin), P(y))
    return y


def rope_bwd(dy, cos, sin, dx_init=None):
    S, H, Dh = dy.shape
    dx = np.empty_like(dy) if dx_init is None else dx_init.copy()
    lib().oracle_rope_bwd(i64(S), i64(H), i64(Dh), P(dy), P(cos), P(sin), P(dx),
                          C.c_int(dx_init is not None))
    return dx


def silu_gate_fwd(g, u):
    y = np.empty_like(g)
    hh = np.empty_like(g)
    lib().oracle_silu_gate_fwd(i64(g.size), P(g), P(u), P(y), P(hh))
    return y, hh


def silu_gate_bwd(g, u, dh, dg_init=None, du_init=None):
    y, _ = silu_gate_fwd(g, u)
    dg = np.empty_like(g) if dg_init is None else dg_init.copy()
    du = np.empty_like(g) if du_init is None else du_init.copy()
    lib().oracle_silu_gate_bwd(i64(g.size), P(g), P(u), P(y), P(dh), P(dg),
                               C.c_int(dg_init is not None), P(du), C.c_int(du_init is not None))
    return dg, du


def causal_softmax_fwd(s16):
    S, H, S2 = s16.shape
    assert S == S2
    p = np.empty_like(s16)
    lib().oracle_causal_softmax_fwd(i64(S), i64(H), P(s16), P(p))
    return p


def causal_softmax_bwd(s16, dp16):
    S, H, _ = s16.shape
    ds = np.empty_like(s16)
    lib().oracle_causal_softmax_bwd(i64(S), i64(H), P(s16), P(dp16), P(ds))
    return ds


def softmax_ce_fwd(logit, tok, want_prob=True):
    N, V = logit.shape
    prob = np.empty((N, V), np.float32) if want_prob else None
    loss = np.empty((N,), np.float32)
    amax = np.empty((N,), np.uint16)
    rc = lib().oracle_softmax_ce_fwd(i64(N), i64(V), P(logit), P(tok), P(prob), P(loss), P(amax))
    if rc:
        raise IndexError("token id out of range at row %d" % (rc - 1))
    return prob, loss, amax


def softmax_ce_bwd(logit, tok, scale):
    N, V = logit.shape
    d = np.empty((N, V), np.float16)
    rc = lib().oracle_softmax_ce_bwd(i64(N), i64(V), P(logit), P(tok), P(scale), P(d))
    if rc:
        raise IndexError("token id out of range at row %d" % (rc - 1))
    return d


def matmul(ta, tb, A, B, alpha=1.0, beta=0.0, C_init=None):
    """C = f16(alpha op(A) op(B) + beta C); A, B 2-d row-major."""
    M, K = (A.shape[1], A.shape[0]) if ta else A.shape
    K2, N = (B.shape[1], B.shape[0]) if tb else B.shape
    assert K == K2
    Cm = np.zeros((M, N), np.float16) if C_init is None else C_init.copy()
    lib().th_matmul_f16(C.c_int(ta), C.c_int(tb), i64(M), i64(N), i64(K), f32(alpha), P(A),
                        i64(A.shape[1]), P(B), i64(B.shape[1]), f32(beta), P(Cm), i64(N))
    return Cm


def block_matmul(ta, tb, nblk, M, N, K, alpha, A, lda, sa, B, ldb, sb, beta, Cm, ldc, sc):
    lib().th_block_matmul_f16(C.c_int(ta), C.c_int(tb), i64(nblk), i64(M), i64(N), i64(K),
                              f32(alpha), P(A), i64(lda), i64(sa), P(B), i64(ldb), i64(sb),
                              f32(beta), P(Cm), i64(ldc), i64(sc))
    return Cm


def attention_fwd(q, k, v, alpha):
    S, H, Dh = q.shape
    s16 = np.empty((S, H, S), np.float16)
    p16 = np.empty((S, H, S), np.float16)
    o = np.empty_like(q)
    lib().oracle_attention_fwd(i64(S), i64(H), i64(Dh), f32(alpha), P(q), P(k), P(v), P(s16),
                               P(p16), P(o))
    return s16, p16, o


def attention_bwd(q, k, v, dO, alpha):
    S, H, Dh = q.shape
    s16, p16, _ = attention_fwd(q, k, v, alpha)
    dq, dk, dv = np.empty_like(q), np.empty_like(q), np.empty_like(q)
    lib().oracle_attention_bwd(i64(S), i64(H), i64(Dh), f32(alpha), P(q), P(k), P(v), P(s16),
                               P(p16), P(dO), P(dq), P(dk), P(dv))
    return dq, dk, dv


def embed_fwd(W, idx):
    V, D = W.shape
    y = np.empty((idx.size, D), np.float16)
    rc = lib().th_outer_select_f16(i64(V), i64(D), P(W), i64(idx.size), P(idx), P(y))
    if rc:
        raise IndexError("token id out of range at position %d" % (rc - 1))
    return y


def embed_bwd(V, idx, dy):
    D = dy.shape[1]
    dW = np.empty((V, D), np.float16)
    lib().vjp_outer_select_f16(i64(V), i64(D), i64(idx.size), P(idx), P(dy), P(dW))
    return dW


def accumulate_f16(a, b):
    y = np.empty_like(a)
    lib().th_add_f16(i64(a.size), P(a), P(b), P(y))
    return y


# --------------------------------------------------------------------------
# whole model

def param_layout(cfg):
    """Ordered (name, shape) list matching the flat parameter block."""
    D, F, V, L = cfg.D, cfg.F, cfg.V, cfg.L
    out = [("embed", (V, D))]
    for l in range(L):
        out += [("l%d.pre_norm" % l, (D,)), ("l%d.q" % l, (D, D)), ("l%d.k" % l, (D, D)),
                ("l%d.v" % l, (D, D)), ("l%d.o" % l, (D, D)), ("l%d.post_norm" % l, (D,)),
                ("l%d.gate" % l, (F, D)), ("l%d.up" % l, (F, D)), ("l%d.down" % l, (D, F))]
    out += [("head_norm", (D,)), ("lm_head", (V, D))]
    return out


def split_params(cfg, flat):
    out, o = {}, 0
    for name, shp in param_layout(cfg):
        n = int(np.prod(shp))
        out[name] = flat[o:o + n].reshape(shp)
        o += n
    assert o == flat.size
    return out


def llama_step(cfg, param, tok, lm_tok, loss_scale, want_grad=True, grad_cached=None):
    """Returns dict(loss [S] f32, logit [S,V] f16, amax [S] u16, grad flat f16 or None).  grad_cached:
    the gradients held from earlier micro-batches, cached before this cycle
    (examples/open_llama_3b_train.rs:334-345): the returned gradients are theirs plus this cycle's."""
    n = lib().oracle_param_elems(C.byref(cfg))
    assert param.size == n and param.dtype == np.float16
    loss = np.empty((cfg.S,), np.float32)
    logit = np.empty((cfg.S, cfg.V), np.float16)
    amax = np.empty((cfg.S,), np.uint16)
    grad = np.zeros((n,), np.float16) if want_grad else None
    if grad_cached is not None:
        assert want_grad and grad_cached.dtype == np.float16 and grad_cached.size == n
        grad = np.array(grad_cached, dtype=np.float16, copy=True, order="C").reshape(n)
    rc = lib().oracle_llama_step(C.byref(cfg), P(param), P(tok), P(lm_tok), P(loss_scale), P(loss),
                                 P(logit), P(amax), P(grad), C.c_int(0 if grad_cached is None else 1))
    if rc:
        raise IndexError("oracle_llama_step failed rc=%d" % rc)
    return dict(loss=loss, logit=logit, amax=amax, grad=grad)


# ---------------------------------------------------------------- numerical-health digests
def nan_count(x):
    """Number of NaNs in an f16 tensor (src/thunk/op.rs:273-349)."""
    x = np.ascontiguousarray(x)
    return int(lib().oracle_nan_count_f16(i64(x.size), P(x)))


def abs_log2_hist8(x):
    """int64[256] histogram of floor(log2 |x|) classes of an f16 tensor (src/thunk/op.rs:351-441)."""
    x = np.ascontiguousarray(x)
    h = np.zeros(256, np.int64)
    lib().oracle_abs_log2_hist8_f16(i64(x.size), P(x), P(h))
    return h


def abs_log2_bin(bits):
    """Histogram bin of one f16 bit pattern."""
    return int(lib().oracle_abs_log2_bin(int(bits)))


# ---------------------------------------------------------------- optimiser thunks
def online_average_scale(u, v, src_scale, rate):
    """v + rate * (src_scale * f32(u) - v) into a copy of v (src/thunk/op.rs:3884-3939)."""
    u = h(u)
    v = np.array(v, dtype=np.float32, copy=True, order="C")
    lib().th_online_average_scale_f16_f32(i64(u.size), P(u), P(v), f32(src_scale), f32(rate))
    return v


def online_average_square_scale(u, v, src_scale, rate):
    """v + rate * ((src_scale * f32(u))^2 - v) into a copy of v (src/thunk/op.rs:3941-4002)."""
    u = h(u)
    v = np.array(v, dtype=np.float32, copy=True, order="C")
    lib().th_online_average_square_scale_f16_f32(i64(u.size), P(u), P(v), f32(src_scale), f32(rate))
    return v


def online_adamw_update(g1, g2, w, signed_lr, lr_unbias, lamda, eps):
    """w + signed_lr * (lr_unbias * (g1 / (sqrt(g2) + eps)) + lamda * w) into a copy of w
    (src/thunk/op.rs:4004-4062)."""
    g1 = np.ascontiguousarray(g1, dtype=np.float32)
    g2 = np.ascontiguousarray(g2, dtype=np.float32)
    w = np.array(w, dtype=np.float32, copy=True, order="C")
    lib().th_online_adamw_update_f32(i64(w.size), P(g1), P(g2), P(w), f32(signed_lr), f32(lr_unbias),
                                     f32(lamda), f32(eps))
    return w


def cast_f32_f16(x):
    """CastFutThunkSpec f32 -> f16, round to nearest even (src/thunk/op.rs:621-663)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    y = np.empty(x.shape, np.float16)
    lib().th_cast_f32_f16(i64(x.size), P(x), P(y))
    return y


def adamw32_scalars(iter_nr, grad_scale, lr, wd, a1, a2, eps):
    """{grad_unscale, a1, a2, signed_lr, lr_unbias, lamda, eps * unbias2} of one AdamW32 step
    (src/librarium/adamw.rs:45-60, src/op.rs:984-1023); grad_scale None or <= 0 = unscaled."""
    out = np.zeros(7, np.float32)
    rc = lib().oracle_adamw32_scalars(int(iter_nr), f32(grad_scale or 0.0), f32(lr), f32(wd), f32(a1), f32(a2),
                                      f32(eps), P(out))
    if rc:
        raise ValueError("adamw32: invalid iter_nr=%d (should be positive)" % iter_nr)
    return out


def adamw32_step(grad, avg, avg2, master, scalars):
    """One step of one tensor: returns new (avg, avg2, master f32, param f16)."""
    grad = h(grad)
    avg, avg2, master = (np.array(x, dtype=np.float32, copy=True, order="C") for x in (avg, avg2, master))
    param = np.empty(grad.shape, np.float16)
    sc = np.ascontiguousarray(scalars, dtype=np.float32)
    lib().oracle_adamw32_step(i64(grad.size), P(grad), P(avg), P(avg2), P(master), P(param), P(sc))
    return avg, avg2, master, param


# ---------------------------------------------------------------- weight ingest
def raw_cast(kind, x):
    """The four bf16 raw casts (src/thunk/op.rs:665-803); bf16 travels as uint16 bit patterns."""
    src, dst = {"bf16_f16": (np.uint16, np.float16), "bf16_f32": (np.uint16, np.float32),
                "f32_bf16": (np.float32, np.uint16), "f16_bf16": (np.float16, np.uint16)}[kind]
    x = np.ascontiguousarray(x, dtype=src)
    y = np.empty(x.shape, dst)
    getattr(lib(), "th_raw_cast_" + kind)(i64(x.size), P(x), P(y))
    return y


def cell_matcher_match(keys, rules):
    """CellMatcher::match_ (src/util/cell.rs:63-112).  rules: tuples of int / str patterns.  Returns,
    per rule, the matched key or None.  The key set is ordered; a matched key leaves it."""
    left = sorted(set(keys), key=lambda k: k.encode())
    out = []
    for pat in rules:
        pat = pat if isinstance(pat, tuple) else (pat,)
        hit = None
        for key in left:
            idx = 0
            for tok in key.split("."):
                p = pat[idx]
                if isinstance(p, int):
                    if tok == "%d" % p:
                        idx += 1
                elif tok == p or p in tok:
                    idx += 1
                if idx == len(pat):
                    break
            if idx == len(pat):
                hit = key
                break
        if hit is not None:
            left.remove(hit)
        out.append(hit)
    return out


def llama_rules(num_layers):
    """The rules of Llama::match_pickle_dir in parameter order (src/librarium/llama.rs:284-302)."""
    rules = [("embed",)]
    for i in range(num_layers):
        rules += [(i, "input_layernorm"), (i, "attn", "q_proj"), (i, "attn", "k_proj"), (i, "attn", "v_proj"),
                  (i, "attn", "o_proj"), (i, "post_attention_layernorm"), (i, "mlp", "gate"), (i, "mlp", "up"),
                  (i, "mlp", "down")]
    return rules + [("norm",), ("lm_head",)]


def read_safetensors_header(path):
    """{name: (dtype string, shape, absolute byte range)} of one safetensors file, from the published
    layout (u64 LE header length, JSON header, data); what TensorsDir::_reopen keeps per tensor
    (src/util/safetensor.rs:88-113)."""
    import json
    import struct
    with open(path, "rb") as f:
        (n,) = struct.unpack("<Q", f.read(8))
        hdr = json.loads(f.read(n).decode("utf-8"))
    out = {}
    for name, e in hdr.items():
        if name == "__metadata__":
            continue
        b, e_ = e["data_offsets"]
        out[name] = (e["dtype"], tuple(e["shape"]), (8 + n + b, 8 + n + e_))
    return out


# ---------------------------------------------------------------- KV-cached forward pass
def llama_cached_state(cfg):
    """Zeroed k / v caches [L, cap, H*Dh] f16 (LlamaCached::init_state, src/librarium/llama.rs:762-782)."""
    shape = (cfg.L, cfg.S, cfg.D)
    return np.zeros(shape, np.float16), np.zeros(shape, np.float16)


def llama_cached_apply(cfg, param, k_cache, v_cache, in_tok, prev, next_, want_prob=False):
    """LlamaCached::apply (src/librarium/llama.rs:805-963) for positions prev .. next_-1; cfg.S is the
    sequence capacity.  Updates k_cache, v_cache and in_tok (the generated token is appended) in
    place; returns dict(logit [T,V] f16, tok [T] u16, prob [T,V] f32 or None)."""
    T = next_ - prev
    assert param.dtype == np.float16 and in_tok.dtype == np.uint16 and in_tok.size == cfg.S
    assert k_cache.flags["C_CONTIGUOUS"] and v_cache.flags["C_CONTIGUOUS"]
    logit = np.empty((T, cfg.V), np.float16)
    prob = np.empty((T, cfg.V), np.float32) if want_prob else None
    tok = np.empty((T,), np.uint16)
    lib().oracle_llama_cached_apply.restype = i64
    rc = lib().oracle_llama_cached_apply(C.byref(cfg), P(param), P(k_cache), P(v_cache), P(in_tok), i64(prev),
                                         i64(next_), P(logit), P(prob), P(tok))
    if rc:
        raise ValueError("oracle_llama_cached_apply: status %d" % rc)
    return dict(logit=logit, tok=tok, prob=prob)

