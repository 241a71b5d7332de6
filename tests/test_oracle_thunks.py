"""Pins the CPU oracle against what the mathematics fixes (no GPU needed).

Each check is chosen so that a plausible mistake in the oracle (dropped term,
wrong sign or index, transposed operand) fails it; none of them retypes the
oracle's own formula.
"""
import numpy as np
import pytest
import scipy.special as sp

from tests.util import f64, rel_l2, max_rel, rng, randn16


# ---------------------------------------------------------------- f16 codec
def test_f16_decode_all_bit_patterns(oracle):
    L = oracle.lib()
    allh = np.arange(65536, dtype=np.uint16)
    got = np.array([L.oracle_h2f(int(v)) for v in allh], dtype=np.float32)
    want = allh.view(np.float16).astype(np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))


def test_f16_encode_rne_ties_subnormals_overflow(oracle):
    L = oracle.lib()
    r = rng(1)
    vals = np.concatenate([
        r.standard_normal(20000).astype(np.float32) * np.float32(10.0) ** r.integers(-9, 5, 20000),
        # exact ties between neighbouring halves, around 1, 2048 and in the subnormal range
        np.array([1 + 2 ** -11, 1 + 3 * 2 ** -11, 2049, 2051, 65519.9, 65520, 65536, 1e9,
                  2 ** -24, 2 ** -25, 1.5 * 2 ** -24, 2.5 * 2 ** -24, 2 ** -14, 2 ** -14 - 2 ** -25,
                  0.0, -0.0, np.inf, -np.inf], dtype=np.float32)])
    vals = np.concatenate([vals, -vals]).astype(np.float32)
    got = np.array([L.oracle_f2h(float(v)) for v in vals], dtype=np.uint16)
    want = vals.astype(np.float16).view(np.uint16)
    assert np.array_equal(got, want)


# ---------------------------------------------------------------- GEMM
@pytest.mark.parametrize("ta,tb", [(0, 0), (0, 1), (1, 0), (1, 1)])
def test_matmul_vs_fp64_bruteforce(oracle, ta, tb):
    r = rng(10 + 2 * ta + tb)
    M, N, K = 13, 21, 37
    A = randn16(r, (K, M) if ta else (M, K))
    B = randn16(r, (N, K) if tb else (K, N))
    C0 = randn16(r, (M, N))
    opA = f64(A).T if ta else f64(A)
    opB = f64(B).T if tb else f64(B)
    for alpha, beta in [(1.0, 0.0), (0.1, 0.0), (1.0, 1.0)]:
        got = oracle.matmul(ta, tb, A, B, alpha, beta, C0)
        want = alpha * (opA @ opB) + beta * f64(C0)
        # fp32 accumulate then one f16 rounding: half an ulp of |want| plus fp32 noise
        assert np.all(np.abs(f64(got) - want) <= 2 ** -11 * np.abs(want) + 1e-4)
        assert got.dtype == np.float16


def test_block_matmul_strided_heads(oracle):
    """Blocks live side by side in [S,H,Dh] / [S,H,S] tensors (strides, not copies)."""
    r = rng(3)
    S, H, Dh = 9, 3, 6
    q, k = randn16(r, (S, H, Dh)), randn16(r, (S, H, Dh))
    s = np.zeros((S, H, S), np.float16)
    oracle.block_matmul(0, 1, H, S, S, Dh, 0.5, q, H * Dh, Dh, k, H * Dh, Dh, 0.0, s, H * S, S)
    want = 0.5 * np.einsum("ihd,jhd->ihj", f64(q), f64(k))
    assert np.all(np.abs(f64(s) - want) <= 2 ** -11 * np.abs(want) + 1e-4)


# ---------------------------------------------------------------- softmax family
def test_softmax_rows_and_closed_form(oracle):
    r = rng(4)
    x = (r.standard_normal((7, 33)) * 3).astype(np.float32)
    y = np.empty_like(x)
    oracle.lib().th_softmax_f32(7, 33, oracle.P(x), oracle.P(y))
    assert np.allclose(y.sum(1), 1.0, atol=1e-6)
    assert np.allclose(y, sp.softmax(f64(x), axis=1), rtol=1e-5, atol=1e-8)
    # equal logits -> 1/n exactly representable for n = 32
    x = np.full((2, 32), 3.25, np.float32)
    y = np.empty_like(x)
    oracle.lib().th_softmax_f32(2, 32, oracle.P(x), oracle.P(y))
    assert np.all(y == np.float32(1 / 32))


def test_softmax_post_adj_is_jacobian_transpose(oracle):
    """J^T dy from central differences of an fp64 softmax."""
    r = rng(5)
    n = 12
    x = r.standard_normal((3, n))
    dy = r.standard_normal((3, n))
    y32 = sp.softmax(x, axis=1).astype(np.float32)
    dy32 = dy.astype(np.float32)
    out = np.empty_like(y32)
    oracle.lib().th_softmax_post_adj_f32(3, n, oracle.P(y32), oracle.P(dy32), oracle.P(out))
    want = np.zeros_like(x)
    h = 1e-6
    for j in range(n):
        e = np.zeros(n); e[j] = h
        d = (sp.softmax(x + e, axis=1) - sp.softmax(x - e, axis=1)) / (2 * h)
        want[:, j] = (d * f64(dy32)).sum(1)
    assert np.allclose(out, want, rtol=1e-4, atol=1e-6)
    assert np.allclose(out.sum(1), 0.0, atol=1e-6)       # adjoint rows sum to zero


def test_nll_is_logsumexp_minus_target(oracle):
    r = rng(6)
    N, V = 9, 50
    x = (r.standard_normal((N, V)) * 4).astype(np.float32)
    k = r.integers(0, V, N).astype(np.uint16)
    out = np.empty(N, np.float32)
    rc = oracle.lib().th_softmax_nll_f32(N, V, oracle.P(x), oracle.P(k), oracle.P(out))
    assert rc == 0
    want = sp.logsumexp(f64(x), axis=1) - f64(x)[np.arange(N), k]
    assert np.allclose(out, want, rtol=1e-5, atol=1e-6)
    k[4] = V                                             # asserted range in the reference
    assert oracle.lib().th_softmax_nll_f32(N, V, oracle.P(x), oracle.P(k), oracle.P(out)) == 5


def test_ce_fwd_bwd(oracle):
    r = rng(7)
    N, V = 11, 64
    logit = randn16(r, (N, V), 2.0)
    tok = r.integers(0, V, N).astype(np.uint16)
    scale = r.random(N).astype(np.float32)
    scale[0] = 0.0
    prob, loss, amax = oracle.softmax_ce_fwd(logit, tok)
    x = f64(logit)
    assert np.allclose(loss, sp.logsumexp(x, 1) - x[np.arange(N), tok], rtol=1e-5, atol=1e-6)
    assert np.allclose(prob, sp.softmax(x, 1), rtol=1e-5, atol=1e-8)
    # argmax: first index of the maximum (ties resolved to the lowest index)
    assert np.array_equal(amax, np.argmax(x, axis=1).astype(np.uint16))
    d = oracle.softmax_ce_bwd(logit, tok, scale)
    # gradient of sum_n scale_n * loss_n by central differences in fp64
    want = np.zeros((N, V))
    h = 1e-5
    for j in range(V):
        e = np.zeros(V); e[j] = h
        lp = sp.logsumexp(x + e, 1) - (x + e)[np.arange(N), tok]
        lm = sp.logsumexp(x - e, 1) - (x - e)[np.arange(N), tok]
        want[:, j] = scale * (lp - lm) / (2 * h)
    assert rel_l2(d, want) < 5e-4 and max_rel(d, want) < 5e-3
    assert np.all(d[0] == 0)                             # zero loss scale -> zero row
    assert np.all(np.abs(f64(d).sum(1)) < 2e-3)          # sum_j (p_j - 1[j=t]) = 0
    with pytest.raises(IndexError):
        oracle.softmax_ce_fwd(logit, np.full(N, V, np.uint16))


def test_ce_saturated_kat(oracle):
    """One logit far above the rest: p = one-hot, loss 0 at the target, d = 0."""
    N, V = 2, 16
    logit = np.zeros((N, V), np.float16)
    logit[:, 3] = 60.0
    tok = np.array([3, 3], np.uint16)
    prob, loss, amax = oracle.softmax_ce_fwd(logit, tok)
    assert np.all(loss == 0) and np.all(amax == 3)
    d = oracle.softmax_ce_bwd(logit, tok, np.ones(N, np.float32))
    assert np.all(d == 0)


def test_arg_max_ties_first_index(oracle):
    logit = np.zeros((1, 8), np.float16)
    logit[0, [2, 5]] = 1.0
    _, _, amax = oracle.softmax_ce_fwd(logit, np.zeros(1, np.uint16))
    assert amax[0] == 2


# ---------------------------------------------------------------- RMSNorm
def _rms_f64(x, w, eps):
    r = np.sqrt((x * x).mean(1, keepdims=True) + eps)
    return w * (x / r)


def test_rmsnorm_fwd_closed_form_and_kat(oracle):
    r = rng(8)
    N, D = 6, 40
    x, w = randn16(r, (N, D)), randn16(r, (D,))
    y, t, s = oracle.rmsnorm_fwd(x, w, 1e-6)
    want = _rms_f64(f64(x), f64(w), 1e-6)
    assert np.all(np.abs(f64(y) - want) <= 2 ** -11 * np.abs(want) * 1.01 + 1e-7)
    # constant row c, unit weight, eps = 0 -> exactly sign(c)
    x = np.full((1, 16), -3.0, np.float16)
    y, _, _ = oracle.rmsnorm_fwd(x, np.ones(16, np.float16), 0.0)
    assert np.all(y == -1.0)


def test_rmsnorm_bwd_vs_fp64_finite_differences(oracle):
    r = rng(9)
    N, D = 5, 24
    x, w, dy = randn16(r, (N, D)), randn16(r, (D,)), randn16(r, (N, D))
    eps = 1e-6
    dx, dw = oracle.rmsnorm_bwd(x, w, eps, dy)
    X, W, G = f64(x), f64(w), f64(dy)
    h = 1e-6
    wdx = np.zeros_like(X)
    for n in range(N):
        for d in range(D):
            e = np.zeros_like(X); e[n, d] = h
            wdx[n, d] = ((_rms_f64(X + e, W, eps) - _rms_f64(X - e, W, eps)) * G).sum() / (2 * h)
    wdw = np.zeros(D)
    for d in range(D):
        e = np.zeros(D); e[d] = h
        wdw[d] = ((_rms_f64(X, W + e, eps) - _rms_f64(X, W - e, eps)) * G).sum() / (2 * h)
    assert rel_l2(dx, wdx) < 1e-3 and max_rel(dx, wdx) < 1e-2
    assert rel_l2(dw, wdw) < 1e-3 and max_rel(dw, wdw) < 1e-2


def test_rmsnorm_bwd_accumulates_in_f16(oracle):
    r = rng(11)
    N, D = 4, 16
    x, w, dy = randn16(r, (N, D)), randn16(r, (D,)), randn16(r, (N, D))
    dx0, dw0 = randn16(r, (N, D)), randn16(r, (D,))
    dx, dw = oracle.rmsnorm_bwd(x, w, 1e-6, dy)
    dxa, dwa = oracle.rmsnorm_bwd(x, w, 1e-6, dy, dx0, dw0)
    assert rel_l2(dxa, f64(dx0) + f64(dx)) < 1e-3
    assert np.array_equal(dwa, (dw0.astype(np.float32) + dw.astype(np.float32)).astype(np.float16))


# ---------------------------------------------------------------- RoPE
def test_rope_tables_vs_library(oracle):
    S, Dh = 64, 20
    cos, sin = oracle.rope_tables(S, Dh)
    i = np.arange(Dh // 2)
    fr = np.arange(S)[:, None] * (10000.0 ** (-2.0 * i / Dh))[None, :]
    fr = np.concatenate([fr, fr], 1)
    assert np.all(np.abs(f64(cos) - np.cos(fr)) < 6e-4)   # one f16 ulp at |v| <= 1, f32 phase
    assert np.all(np.abs(f64(sin) - np.sin(fr)) < 6e-4)
    assert np.all(cos[0] == 1) and np.all(sin[0] == 0)    # position 0 is the identity
    assert np.array_equal(cos[:, :Dh // 2], cos[:, Dh // 2:])


def test_rope_position_zero_identity_and_rotation(oracle):
    r = rng(12)
    S, H, Dh = 5, 2, 8
    x = randn16(r, (S, H, Dh))
    cos, sin = oracle.rope_tables(S, Dh)
    y = oracle.rope_fwd(x, cos, sin)
    assert np.array_equal(y[0], x[0])
    # a quarter turn (cos 0, sin 1): y = rot(x) = [-x_r, x_l] exactly
    c0 = np.zeros((S, Dh), np.float16); s1 = np.ones((S, Dh), np.float16)
    y = oracle.rope_fwd(x, c0, s1)
    assert np.array_equal(y[..., :4], -x[..., 4:]) and np.array_equal(y[..., 4:], x[..., :4])


def test_rope_bwd_is_exact_transpose(oracle):
    """<rope(x), dy> == <x, rope_adj(dy)> exactly when every product is representable."""
    r = rng(13)
    S, H, Dh = 6, 3, 8
    x = r.integers(-8, 9, (S, H, Dh)).astype(np.float16)
    dy = r.integers(-8, 9, (S, H, Dh)).astype(np.float16)
    tab_vals = np.array([0, 0.5, -0.5, 1, -1, 2, 0.25], np.float16)
    cos = r.choice(tab_vals, (S, Dh)).astype(np.float16)   # the transpose property holds for any table
    sin = r.choice(tab_vals, (S, Dh)).astype(np.float16)
    y = oracle.rope_fwd(x, cos, sin)
    dx = oracle.rope_bwd(dy, cos, sin)
    assert (f64(y) * f64(dy)).sum() == (f64(x) * f64(dx)).sum()
    # accumulate mode adds the previous value
    dx0 = r.integers(-4, 5, (S, H, Dh)).astype(np.float16)
    assert np.array_equal(oracle.rope_bwd(dy, cos, sin, dx0), dx0 + dx)


# ---------------------------------------------------------------- SiLU gate
def test_silu_gate_fwd_bwd_textbook(oracle):
    r = rng(14)
    n = 4096
    g, u, dh = randn16(r, (n,), 2.0), randn16(r, (n,)), randn16(r, (n,))
    y, hh = oracle.silu_gate_fwd(g, u)
    G, U, DH = f64(g), f64(u), f64(dh)
    sig = sp.expit(G)
    assert rel_l2(hh, G * sig * U) < 6e-4
    dg, du = oracle.silu_gate_bwd(g, u, dh)
    assert rel_l2(du, DH * G * sig) < 6e-4
    want_dg = DH * U * sig * (1 + G * (1 - sig))          # textbook d silu
    assert rel_l2(dg, want_dg) < 1e-3 and max_rel(dg, want_dg) < 1e-2
    # silu(0) = 0, derivative 1/2
    z = np.zeros(4, np.float16); one = np.ones(4, np.float16)
    dg, du = oracle.silu_gate_bwd(z, one, one)
    assert np.all(dg == 0.5) and np.all(du == 0)


# ---------------------------------------------------------------- causal softmax
def test_causal_softmax_fwd_bwd(oracle):
    r = rng(15)
    S, H = 10, 3
    s16 = randn16(r, (S, H, S))
    p = oracle.causal_softmax_fwd(s16)
    iu = np.triu_indices(S, 1)
    assert np.all(p[iu[0], :, iu[1]] == 0)                # strictly upper triangle is exactly 0
    assert np.all(p[0, :, 0] == 1)
    X = f64(s16).copy()
    mask = np.arange(S)[:, None, None] < np.arange(S)[None, None, :]
    Xm = np.where(mask, -np.inf, X)
    want = sp.softmax(Xm, axis=2)
    assert np.all(np.abs(f64(p) - want) <= 2 ** -11 * want * 1.01 + 1e-7)
    dp = randn16(r, (S, H, S))
    ds = oracle.causal_softmax_bwd(s16, dp)
    assert np.all(ds[iu[0], :, iu[1]] == 0)
    t = want * f64(dp)
    wds = t - t.sum(2, keepdims=True) * want
    wds = np.where(mask, 0.0, wds)
    assert rel_l2(ds, wds) < 6e-4
    # finite differences on one row pin the closed form itself
    i, hd = 6, 1
    hstep = 1e-6
    fd = np.zeros(S)
    for j in range(i + 1):
        e = np.zeros(S); e[j] = hstep
        pp = sp.softmax(np.where(np.arange(S) > i, -np.inf, X[i, hd] + e))
        pm = sp.softmax(np.where(np.arange(S) > i, -np.inf, X[i, hd] - e))
        fd[j] = ((pp - pm) / (2 * hstep) * f64(dp)[i, hd]).sum()
    assert np.allclose(fd, wds[i, hd], atol=1e-6)


# ---------------------------------------------------------------- embedding
def test_embedding_gather_scatter(oracle):
    r = rng(16)
    V, D, S = 12, 8, 20
    W = randn16(r, (V, D))
    idx = r.integers(0, V, S).astype(np.uint16)
    y = oracle.embed_fwd(W, idx)
    assert np.array_equal(y.view(np.uint16), W[idx].view(np.uint16))     # bit-exact gather
    dy = randn16(r, (S, D))
    dW = oracle.embed_bwd(V, idx, dy)
    want = np.zeros((V, D)); np.add.at(want, idx, f64(dy))
    assert np.array_equal(dW, want.astype(np.float16))
    never = np.setdiff1d(np.arange(V), idx)
    assert np.all(dW[never] == 0)
    with pytest.raises(IndexError):
        oracle.embed_fwd(W, np.array([V], np.uint16))


# ---------------------------------------------------------------- attention block
def test_attention_bwd_vs_fp64_autograd_free_closed_form(oracle):
    """dQ, dK, dV of causal attention from the fp64 closed form (independent einsum code)."""
    r = rng(17)
    S, H, Dh = 12, 2, 8
    alpha = 1 / np.sqrt(Dh)
    q, k, v, dO = (randn16(r, (S, H, Dh)) for _ in range(4))
    dq, dk, dv = oracle.attention_bwd(q, k, v, dO, alpha)
    Q, K, Vv, DO = f64(q), f64(k), f64(v), f64(dO)
    Sc = alpha * np.einsum("ihd,jhd->hij", Q, K)
    mask = np.arange(S)[:, None] < np.arange(S)[None, :]
    Sc = np.where(mask[None], -np.inf, Sc)
    Pm = sp.softmax(Sc, axis=2)
    dV = np.einsum("hij,ihd->jhd", Pm, DO)
    dP = np.einsum("ihd,jhd->hij", DO, Vv)
    dS = Pm * (dP - (Pm * dP).sum(2, keepdims=True))
    dQ = alpha * np.einsum("hij,jhd->ihd", dS, K)
    dK = alpha * np.einsum("hij,ihd->jhd", dS, Q)
    for got, want in ((dq, dQ), (dk, dK), (dv, dV)):
        assert rel_l2(got, want) < 2e-3 and max_rel(got, want) < 2e-2
