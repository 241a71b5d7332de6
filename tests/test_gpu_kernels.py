"""Parity of every HIP kernel against the CPU oracle on the same seeded inputs (MI355X).

All calls go through the C ABI (cacti_amd.ops is a thin ctypes layer).  Tolerances:
tests/util.py (rel-L2 <= 1e-3, max element relative error <= 2e-2); gather / argmax /
index results bit-exact.  Elementwise kernels reproduce the oracle's rounding points, so
most of them are in fact compared bit for bit (`exact_frac`).
"""
import numpy as np
import pytest
import torch

from tests.util import assert_parity, rng, randn16

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    from cacti_amd import ops as o
    return o


def dev(a):
    if a.dtype == np.uint16:
        a = a.view(np.int16)
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    a = t.detach().cpu().numpy()
    return a


def exact_frac(a, b):
    return float(np.mean(a.view(np.uint16) == b.view(np.uint16)))


def assert_bits(a, b, name=""):
    """Bit-for-bit equality of two f16 arrays, with a short message instead of an array dump."""
    eq = a.view(np.uint16) == b.view(np.uint16)
    assert eq.all(), "%s: %d of %d elements differ" % (name, int((~eq).sum()), eq.size)


def say(*a):
    print(*a, flush=True)


# ---------------------------------------------------------------- wave reduce
def test_wave_reduce_selftest(ops):
    s, rs, m, cnt = ops.selftest_wave_reduce()
    assert s == rs and cnt == 64.0, (s, rs, m, cnt)


# ---------------------------------------------------------------- RMSNorm
@pytest.mark.parametrize("N,D", [(2048, 3200), (128, 256), (37, 4096), (5, 8), (16, 8192)])
def test_rms_norm_fwd(ops, oracle, N, D):
    say("rms_norm_fwd", N, D)
    r = rng(100 + D)
    x, w = randn16(r, (N, D)), randn16(r, (D,))
    want, _, _ = oracle.rmsnorm_fwd(x, w, 1e-6)
    got = host(ops.rms_norm_fwd(dev(x), dev(w), 1e-6))
    assert_parity(got, want, "rms_norm_fwd")
    assert exact_frac(got, want) > 0.999


@pytest.mark.parametrize("N,D", [(2048, 3200), (37, 4096), (5, 8)])
def test_add_rms_norm_fwd_equals_the_two_thunks(ops, oracle, N, D):
    """One launch for x = a + b and rms_norm(x): bit for bit the add thunk followed by the norm."""
    say("add_rms_norm_fwd", N, D)
    r = rng(120 + N)
    a, b, w = randn16(r, (N, D)), randn16(r, (N, D)), (randn16(r, (D,), 0.1) + np.float16(1))
    s, y = ops.add_rms_norm_fwd(dev(a), dev(b), dev(w), 1e-6)
    want_s = oracle.accumulate_f16(a, b)
    assert_bits(host(s), want_s, "sum")
    assert_bits(host(y), host(ops.rms_norm_fwd(dev(want_s), dev(w), 1e-6)), "norm vs unfused kernel")
    assert_parity(host(y), oracle.rmsnorm_fwd(want_s, w, 1e-6)[0], "norm vs oracle")


@pytest.mark.parametrize("N,D", [(2048, 3200), (128, 256), (37, 4096), (5, 8), (16, 8192)])
@pytest.mark.parametrize("acc", [False, True])
def test_rms_norm_bwd(ops, oracle, N, D, acc):
    say("rms_norm_bwd", N, D, acc)
    r = rng(200 + D + acc)
    x, w, dy = randn16(r, (N, D)), randn16(r, (D,)), randn16(r, (N, D))
    dx0 = randn16(r, (N, D)) if acc else None
    dw0 = randn16(r, (D,)) if acc else None
    wdx, wdw = oracle.rmsnorm_bwd(x, w, 1e-6, dy, dx0, dw0)
    gdx, gdw = ops.rms_norm_bwd(dev(x), dev(w), 1e-6, dev(dy), dev(dx0) if acc else None,
                                dev(dw0) if acc else None)
    assert_parity(host(gdx), wdx, "dx")
    assert_parity(host(gdw), wdw, "dw")
    assert exact_frac(host(gdx), wdx) > 0.99


# ---------------------------------------------------------------- RoPE
def test_rope_tables(ops, oracle):
    for S, Dh in [(2048, 100), (128, 64)]:
        c, s = ops.rope_tables(S, Dh)
        wc, ws = oracle.rope_tables(S, Dh)
        # device cos/sin/pow differ from libm in the last ulp of f32: allow one f16 ulp
        assert np.max(np.abs(host(c).astype(np.float32) - wc.astype(np.float32))) <= 2 ** -10
        assert np.max(np.abs(host(s).astype(np.float32) - ws.astype(np.float32))) <= 2 ** -10
        assert exact_frac(host(c), wc) > 0.99 and exact_frac(host(s), ws) > 0.99


@pytest.mark.parametrize("S,H,Dh", [(2048, 32, 100), (128, 4, 64), (7, 2, 12), (33, 32, 100)])
def test_rope_fwd_bwd(ops, oracle, S, H, Dh):
    say("rope", S, H, Dh)
    r = rng(300 + S)
    x, dy, dx0 = randn16(r, (S, H, Dh)), randn16(r, (S, H, Dh)), randn16(r, (S, H, Dh))
    cos, sin = oracle.rope_tables(S, Dh)
    dc, ds = dev(cos), dev(sin)
    assert_bits(host(ops.rope_fwd(dev(x), dc, ds)), oracle.rope_fwd(x, cos, sin), "fwd")
    assert_bits(host(ops.rope_bwd(dev(dy), dc, ds)), oracle.rope_bwd(dy, cos, sin), "bwd")
    assert_bits(host(ops.rope_bwd(dev(dy), dc, ds, dev(dx0))), oracle.rope_bwd(dy, cos, sin, dx0),
                "bwd+")


def test_rope_bwd_in_place(ops, oracle):
    r = rng(310)
    S, H, Dh = 64, 32, 100
    dy = randn16(r, (S, H, Dh))
    cos, sin = oracle.rope_tables(S, Dh)
    t, dc, ds = dev(dy), dev(cos), dev(sin)
    from cacti_amd import ffi
    ffi.call("cacti_hip_rope_bwd", S, H, Dh, t.data_ptr(), dc.data_ptr(), ds.data_ptr(),
             t.data_ptr(), 0, torch.cuda.current_stream().cuda_stream)
    assert_bits(host(t), oracle.rope_bwd(dy, cos, sin), "in place")


# ---------------------------------------------------------------- SiLU gate
@pytest.mark.parametrize("shape", [(2048, 8640), (128, 688), (1, 8)])
def test_silu_gate(ops, oracle, shape):
    say("silu_gate", shape)
    r = rng(400 + shape[1])
    g, u, dh = randn16(r, shape, 2.0), randn16(r, shape), randn16(r, shape)
    _, wh = oracle.silu_gate_fwd(g, u)
    gh = host(ops.silu_gate_fwd(dev(g), dev(u)))
    assert_parity(gh, wh, "h")
    assert exact_frac(gh, wh) > 0.999
    wdg, wdu = oracle.silu_gate_bwd(g, u, dh)
    gdg, gdu = ops.silu_gate_bwd(dev(g), dev(u), dev(dh))
    assert_parity(host(gdg), wdg, "dg"), assert_parity(host(gdu), wdu, "du")
    assert exact_frac(host(gdg), wdg) > 0.999 and exact_frac(host(gdu), wdu) > 0.999
    dg0, du0 = randn16(r, shape), randn16(r, shape)
    wdg, wdu = oracle.silu_gate_bwd(g, u, dh, dg0, du0)
    gdg, gdu = ops.silu_gate_bwd(dev(g), dev(u), dev(dh), dev(dg0), dev(du0))
    assert_parity(host(gdg), wdg, "dg+"), assert_parity(host(gdu), wdu, "du+")


# ---------------------------------------------------------------- causal softmax
@pytest.mark.parametrize("S,H", [(128, 4), (512, 3), (8, 1), (2048, 2), (640, 2)])
def test_causal_softmax(ops, oracle, S, H):
    say("causal_softmax", S, H)
    r = rng(500 + S)
    s16, dp = randn16(r, (S, H, S), 2.0), randn16(r, (S, H, S), 3.0)
    # the kernels read j <= i only (entries above the diagonal may hold anything) and write
    # j <= i plus zeros up to the next multiple of 256 columns; the rest stays untouched
    i, j = np.arange(S)[:, None, None], np.arange(S)[None, None, :]
    upper = np.broadcast_to(j > i, s16.shape)
    written = np.broadcast_to(j < np.minimum(S, (i + 256) // 256 * 256), s16.shape)
    junk = s16.copy(); junk[upper] = np.float16(np.nan)
    wp = oracle.causal_softmax_fwd(s16)
    out = torch.full((S, H, S), 7.0, dtype=torch.float16, device="cuda")
    from cacti_amd import ffi
    dj = dev(junk)
    ffi.call("cacti_hip_causal_softmax_fwd", S, H, dj.data_ptr(), out.data_ptr(),
             torch.cuda.current_stream().cuda_stream)
    gp = host(out)
    assert np.all(gp[~written] == 7.0) and np.all(gp[written & upper] == 0)
    assert_parity(np.where(written, gp, 0), wp, "p16")
    wds = oracle.causal_softmax_bwd(s16, dp)
    djp = dp.copy(); djp[upper] = np.float16(np.nan)
    ddp = dev(djp)
    out = torch.full((S, H, S), 7.0, dtype=torch.float16, device="cuda")
    ffi.call("cacti_hip_causal_softmax_bwd", S, H, dj.data_ptr(), ddp.data_ptr(), out.data_ptr(),
             torch.cuda.current_stream().cuda_stream)
    gds = host(out)
    assert np.all(gds[~written] == 7.0) and np.all(gds[written & upper] == 0)
    assert_parity(np.where(written, gds, 0), wds, "ds16")


# ---------------------------------------------------------------- softmax cross-entropy
@pytest.mark.parametrize("N,V", [(64, 32000), (128, 1024), (3, 8), (5, 40000)])
def test_softmax_ce(ops, oracle, N, V):
    say("softmax_ce", N, V)
    r = rng(600 + V)
    logit = randn16(r, (N, V), 2.0)
    tok = r.integers(0, V, N).astype(np.uint16)
    scale = r.random(N).astype(np.float32)
    scale[0] = 0.0
    wprob, wloss, wamax = oracle.softmax_ce_fwd(logit, tok)
    gprob, gloss, gamax = ops.softmax_ce_fwd(dev(logit), dev(tok))
    assert_parity(host(gprob), wprob, "prob", l2=1e-5, mx=1e-4)
    assert_parity(host(gloss), wloss, "loss", l2=1e-5, mx=1e-4)
    assert (host(gamax).view(np.uint16) == wamax).all()                # index work: bit-exact
    wd = oracle.softmax_ce_bwd(logit, tok, scale)
    gd = host(ops.softmax_ce_bwd(dev(logit), dev(tok), dev(scale)))
    assert_parity(gd, wd, "dlogit")
    assert gd.size < 10000 or exact_frac(gd, wd) > 0.995
    assert np.all(gd[0] == 0)
    d0 = randn16(r, (N, V), 0.01)
    ga = host(ops.softmax_ce_bwd(dev(logit), dev(tok), dev(scale), dev(d0)))
    assert_parity(ga, oracle.accumulate_f16(d0, wd), "dlogit+")


def test_softmax_ce_argmax_ties_and_bad_token(ops, oracle):
    logit = np.zeros((2, 64), np.float16)
    logit[0, [9, 40]] = 2.0
    logit[1, 63] = 1.0
    tok = np.array([1, 2], np.uint16)
    _, _, amax = ops.softmax_ce_fwd(dev(logit), dev(tok), want_prob=False)
    assert host(amax).view(np.uint16).tolist() == [9, 63]
    with pytest.raises(IndexError):
        ops.softmax_ce_fwd(dev(logit), dev(np.array([1, 64], np.uint16)))


# ---------------------------------------------------------------- embedding
@pytest.mark.parametrize("V,D,S", [(32000, 3200, 2048), (1024, 256, 128), (16, 8, 50)])
def test_embedding(ops, oracle, V, D, S):
    say("embedding", V, D, S)
    r = rng(700 + V)
    W = randn16(r, (V, D), 0.02)
    tok = r.integers(0, V, S).astype(np.uint16)
    tok[S // 2] = tok[0]                                   # force a repeated id
    got = host(ops.embed_fwd(dev(W), dev(tok)))
    assert_bits(got, oracle.embed_fwd(W, tok), "gather")
    dy = randn16(r, (S, D))
    want = oracle.embed_bwd(V, tok, dy)
    got = host(ops.embed_bwd(V, dev(tok), dev(dy)))
    assert_parity(got, want, "dW")
    assert exact_frac(got, want) > 0.9999
    never = np.setdiff1d(np.arange(V), tok)
    assert np.all(got[never] == 0)
    bad = tok.copy()
    bad[1] = V
    with pytest.raises(IndexError):
        ops.embed_fwd(dev(W), dev(bad))


# ---------------------------------------------------------------- accumulate / add
def test_accumulate_and_add(ops, oracle):
    r = rng(800)
    a, b = randn16(r, (100003,)), randn16(r, (100003,))
    got = host(ops.add_f16(dev(a), dev(b)))
    assert_bits(got, oracle.accumulate_f16(a, b), "add")
    t, tb = dev(a), dev(b)
    ops.accumulate_1d(t, tb)
    assert_bits(host(t), oracle.accumulate_f16(a, b), "accumulate")
    f, g = r.standard_normal(1000).astype(np.float32), r.standard_normal(1000).astype(np.float32)
    t, tg = dev(f), dev(g)
    ops.accumulate_1d(t, tg)
    assert (host(t) == f + g).all()
    u, v = r.integers(0, 30000, 1000).astype(np.uint16), r.integers(0, 30000, 1000).astype(np.uint16)
    t, tv = dev(u), dev(v)
    ops.accumulate_1d(t, tv)
    assert (host(t).view(np.uint16) == (u + v).astype(np.uint16)).all()


# ---------------------------------------------------------------- GEMM
GEMM_SHAPES = [
    (128, 128, 32), (256, 384, 192), (100, 72, 40), (128, 688, 256), (128, 256, 688),
    (61, 35, 27),            # nothing aligned: scalar path
    (64, 100, 64), (64, 64, 100),   # head_dim 100: 8-byte path
    (200, 264, 128), (300, 648, 100), (132, 140, 12),   # short K: several column tiles, ragged edges
]


@pytest.mark.parametrize("ta,tb", [(0, 0), (0, 1), (1, 0), (1, 1)])
@pytest.mark.parametrize("M,N,K", GEMM_SHAPES)
def test_gemm_small(ops, oracle, ta, tb, M, N, K):
    say("gemm", ta, tb, M, N, K)
    r = rng(900 + M + 3 * N + 7 * K + 2 * ta + tb)
    A = randn16(r, (K, M) if ta else (M, K))
    B = randn16(r, (N, K) if tb else (K, N))
    C0 = randn16(r, (M, N))
    for alpha, beta in [(1.0, 0.0), (0.1, 1.0)]:
        want = oracle.matmul(ta, tb, A, B, alpha, beta, C0)
        c = dev(C0)
        got = host(ops.gemm(dev(A), dev(B), bool(ta), bool(tb), alpha, beta, c))
        assert_parity(got, want, "gemm")
        assert exact_frac(got, want) > 0.98


# shapes that reach the direct-to-LDS kernels (outputs of at least 1024 x 1024, 16-byte aligned,
# K % 64 == 0) with ragged last tiles in both directions, the 256 x 256 and 256 x 192 wgrad tiles,
# and the forward product whose last columns go to a second launch of small tiles
DIRECT_SHAPES = [
    (0, 1, 1096, 1032, 192), (0, 0, 1096, 1032, 192), (1, 0, 1096, 1032, 128), (1, 1, 1032, 1096, 64),
    (1, 0, 2056, 2304, 64),      # 256 x 256 tiles
    (1, 0, 3200, 3200, 64),      # 256 x 192 tiles
    (0, 1, 1024, 8640, 64),      # 64 full-round column tiles + 448 columns on 64 x 64 tiles
    # the same with 5 .. 13 k tiles: the small tiles load five k tiles ahead (shorter than the
    # pipeline, exactly as long, every length of the peeled tail)
    (0, 1, 1024, 8640, 320), (0, 0, 1024, 8640, 384), (0, 1, 1024, 8640, 448), (0, 0, 1024, 8640, 512),
    (0, 1, 1024, 8640, 576), (0, 0, 1024, 8640, 640), (0, 1, 1024, 8640, 704), (0, 0, 1024, 8640, 832),
    (0, 1, 2048, 24584, 64),     # forward product with at least 768 tiles of 256 x 256
]


@pytest.mark.parametrize("ta,tb,M,N,K", DIRECT_SHAPES)
def test_gemm_direct_load_kernels(ops, oracle, ta, tb, M, N, K):
    say("gemm direct", ta, tb, M, N, K)
    r = rng(970 + M + N + K + 2 * ta + tb)
    A = randn16(r, (K, M) if ta else (M, K))
    B = randn16(r, (N, K) if tb else (K, N), 0.1)
    C0 = randn16(r, (M, N))
    for alpha, beta in [(1.0, 0.0), (0.5, 1.0)]:
        want = oracle.matmul(ta, tb, A, B, alpha, beta, C0)
        got = host(ops.gemm(dev(A), dev(B), bool(ta), bool(tb), alpha, beta, dev(C0)))
        assert_parity(got, want, "gemm direct")
        assert exact_frac(got, want) > 0.98


# one to four rows against a weight matrix (decoding): the streaming kernel, including a row count
# of columns that is not a multiple of its 4 rows per workgroup, a short K, and a padded weight matrix
SKINNY_SHAPES = [(1, 3200, 3200, 0), (2, 8640, 3200, 0), (3, 3200, 8640, 8), (4, 1000, 136, 0), (1, 32000, 3200, 0),
                 (4, 24, 136, 16)]


@pytest.mark.parametrize("M,N,K,pad", SKINNY_SHAPES)
def test_gemm_few_rows_streams_the_weights(ops, oracle, M, N, K, pad):
    say("gemm skinny", M, N, K, pad)
    r = rng(400 + M + N + K)
    A = randn16(r, (M, K))
    Bp = randn16(r, (N, K + pad), 0.05)
    B = Bp[:, :K]
    for alpha in (1.0, 0.125):
        want = oracle.matmul(0, 1, A, np.ascontiguousarray(B), alpha, 0.0, None)
        got = host(ops.gemm(dev(A), dev(Bp)[:, :K], False, True, alpha, 0.0))
        assert_parity(got, want, "gemm skinny")
        assert exact_frac(got, want) > 0.98


@pytest.mark.parametrize("ta,tb,n,M,N,K,off", [(0, 1, 3, 1032, 1096, 192, 0), (1, 0, 2, 1096, 1032, 128, 0), (0, 0, 5, 1024, 1024, 192, 0),
                                             (0, 1, 3, 1032, 1096, 192, 4), (0, 1, 2, 64, 72, 40, 0)])
def test_gemm_pointer_array_batch(ops, oracle, ta, tb, n, M, N, K, off):
    """Products of one shape on separate arrays: one launch for up to four of them (direct-load
    tiles, ragged edges), one after another when an operand is not 16-byte aligned (off) or the
    shape is small; every block against the oracle, with and without accumulation."""
    say("gemm batched", ta, tb, n, M, N, K, off)
    r = rng(300 + n + M + K + off)
    As = [randn16(r, (K, M) if ta else (M, K)) for _ in range(n)]
    Bs = [randn16(r, (N, K) if tb else (K, N), 0.1) for _ in range(n)]
    C0 = [randn16(r, (M, N)) for _ in range(n)]
    shared_a = dev(As[0])

    def place(x):                        # device copy starting `off` elements past an aligned address
        buf = torch.empty(x.size + 8, dtype=torch.float16, device="cuda")
        v = buf[off:off + x.size].view(x.shape)
        v.copy_(dev(x))
        return v
    for alpha, beta in [(1.0, 0.0), (0.5, 1.0)]:
        dA = [shared_a if z == 0 else place(As[z]) for z in range(n)]
        dB = [place(Bs[z]) for z in range(n)]
        dC = [dev(C0[z]) for z in range(n)]
        ops.gemm_batched(dA, dB, bool(ta), bool(tb), alpha, beta, dC)
        for z in range(n):
            want = oracle.matmul(ta, tb, As[z], Bs[z], alpha, beta, C0[z])
            assert_parity(host(dC[z]), want, "gemm batched %d" % z)
            single = host(ops.gemm(dA[z], dB[z], bool(ta), bool(tb), alpha, beta, dev(C0[z])))
            assert np.array_equal(host(dC[z]).view(np.uint16), single.view(np.uint16)), z


@pytest.mark.parametrize("case", ["fwd", "dgrad", "wgrad"])
def test_gemm_projection_shapes(ops, oracle, case):
    """The three GEMMs of one projection at a reduced token count (oracle finishes in seconds)."""
    say("gemm projection", case)
    r = rng(950)
    T, Din, Dout = 256, 3200, 8640
    x, W, dy = randn16(r, (T, Din)), randn16(r, (Dout, Din), 0.02), randn16(r, (T, Dout))
    if case == "fwd":
        got, want = ops.gemm(dev(x), dev(W), False, True), oracle.matmul(0, 1, x, W)
    elif case == "dgrad":
        got, want = ops.gemm(dev(dy), dev(W), False, False), oracle.matmul(0, 0, dy, W)
    else:
        got, want = ops.gemm(dev(dy), dev(x), True, False), oracle.matmul(1, 0, dy, x)
    assert_parity(host(got), want, case)


def test_gemm_linearity_full_size(ops):
    """At full size (no oracle): (A1 + A2) B == A1 B + A2 B up to rounding, against fp32 torch."""
    say("gemm full size")
    torch.manual_seed(0)
    M, N, K = 2048, 3200, 3200
    A = torch.randn(M, K, device="cuda").half()
    B = (torch.randn(N, K, device="cuda") * 0.02).half()
    got = ops.gemm(A, B, False, True)
    ref = (A.float() @ B.float().T)
    err = (got.float() - ref).norm() / ref.norm()
    assert err < 5e-4, err
    got = ops.gemm(A, got, True, False)          # [K,M]^T... (K x N) wgrad-shaped product
    ref = (A.float().T @ ref.half().float())
    assert (got.float() - ref).norm() / ref.norm() < 5e-4


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_gemm_random_shapes_through_the_tile_choice(ops, seed):
    """Seeded random shapes, transpositions and alpha / beta through the automatic choice of kernel and
    tile (direct-load and register tiles, the two-launch column split, the short-K and few-row kernels,
    the element-wise fallback for unaligned operands) against fp32 torch: rel-L2 <= 6e-4 and largest
    error <= 4e-3 of the largest value (f16 rounding of the result is 4.9e-4 relative)."""
    import random
    rnd = random.Random(seed)
    torch.manual_seed(seed)
    for it in range(24):
        ta, tb = rnd.random() < 0.5, rnd.random() < 0.5
        step = rnd.choice([8, 8, 8, 4, 1])                     # alignment class of the leading dimensions
        M = rnd.randrange(1024, 4300, step)
        N = rnd.randrange(1024, 9000, step)
        K = rnd.choice([rnd.randrange(64, 1100, 64), rnd.randrange(8, 600, step), 100])
        if rnd.random() < 0.2:
            N = rnd.choice([3200, 8640, 8192 + 8, 8448])
        if rnd.random() < 0.2:
            M = rnd.choice([2048, 3200, 2056, 1, 3, 4])
        alpha, beta = rnd.choice([1.0, 0.5]), rnd.choice([0.0, 1.0])
        say("gemm random", seed, it, ta, tb, M, N, K, alpha, beta)
        A = torch.randn((K, M) if ta else (M, K), device="cuda").half()
        B = (torch.randn((N, K) if tb else (K, N), device="cuda") * 0.1).half()
        C0 = torch.randn(M, N, device="cuda").half()
        got = ops.gemm(A, B, ta, tb, alpha, beta, C0.clone()).float()
        ref = alpha * ((A.float().T if ta else A.float()) @ (B.float().T if tb else B.float())) + beta * C0.float()
        err = ((got - ref).norm() / ref.norm()).item()
        mx = ((got - ref).abs().max() / ref.abs().max()).item()
        assert err < 6e-4 and mx < 4e-3, (ta, tb, M, N, K, alpha, beta, err, mx)


def test_gemm_colmajor_entry(ops, oracle):
    """The cuBLAS-shaped entry: row-major callers pass operands swapped (thunk/op.rs:4469-4491)."""
    import ctypes as C
    from cacti_amd import ffi
    r = rng(960)
    M, N, K = 96, 80, 64
    x, W = randn16(r, (M, K)), randn16(r, (N, K))
    want = oracle.matmul(0, 1, x, W)             # row-major y = x W^T
    y = torch.empty((M, N), dtype=torch.float16, device="cuda")
    one, zero = C.c_float(1.0), C.c_float(0.0)
    # column-major: y^T (N x M) = W (as col-major K x N, transposed) * x (col-major K x M)
    dW, dx = dev(W), dev(x)
    ffi.call("cacti_hip_gemm_colmajor_f16", 1, 0, N, M, K, C.byref(one), dW.data_ptr(), K,
             dx.data_ptr(), K, C.byref(zero), y.data_ptr(), N,
             torch.cuda.current_stream().cuda_stream)
    assert_parity(host(y), want, "colmajor")


# ---------------------------------------------------------------- attention block
@pytest.mark.parametrize("ta", [0, 1])
def test_head_slab_products_accumulate_in_place(ops, oracle, ta):
    """C[:, h, :] += op(A_h) B[:, h, :] on [S, H, 100] slabs (every other head starts 8 bytes off a
    16-byte boundary): each head's 100 columns get exactly its own product, nothing else moves."""
    say("head slabs accumulate", ta)
    S, H, Dh = 256, 4, 100
    r = rng(1100 + ta)
    a = randn16(r, (S, H, S), 0.1)
    b, c0 = randn16(r, (S, H, Dh)), randn16(r, (S, H, Dh))
    want = np.empty_like(c0)
    for h in range(H):
        want[:, h, :] = oracle.matmul(ta, 0, np.ascontiguousarray(a[:, h, :]),
                                      np.ascontiguousarray(b[:, h, :]), 0.5, 1.0,
                                      np.ascontiguousarray(c0[:, h, :]))
    c = dev(c0)
    ops.gemm_strided_batched(bool(ta), False, H, S, Dh, S, 0.5, dev(a), H * S, S, dev(b), H * Dh, Dh,
                             1.0, c, H * Dh, Dh)
    assert_parity(host(c), want, "slab accumulate")


@pytest.mark.parametrize("S,H,Dh", [(128, 4, 64), (256, 3, 100), (1024, 2, 100), (512, 4, 100), (384, 6, 100)])
@pytest.mark.parametrize("tri", [False, True])
def test_attention_block_via_thunks(ops, oracle, S, H, Dh, tri):
    """Q K^T -> causal softmax -> P V and the adjoint, composed as the reference stages them;
    tri: the products skip the half that the causal mask discards."""
    say("attention", S, H, Dh, tri)
    r = rng(1000 + S)
    alpha = float(np.float32(1.0) / np.sqrt(np.float32(Dh)))
    q, k, v, dO = (randn16(r, (S, H, Dh)) for _ in range(4))
    ws16, wp16, wo = oracle.attention_fwd(q, k, v, alpha)
    dq_, dk_, dv_ = oracle.attention_bwd(q, k, v, dO, alpha)
    Q, K_, V_, DO = dev(q), dev(k), dev(v), dev(dO)
    low = np.broadcast_to(np.arange(S)[:, None, None] >= np.arange(S)[None, None, :], ws16.shape)
    s16 = ops.block_matmul_qk(Q, K_, alpha, causal=tri)
    assert_parity(np.where(low, host(s16), 0), np.where(low, ws16, 0), "s16")
    p16 = ops.causal_softmax_fwd(s16)
    assert_parity(np.where(low, host(p16), 0), wp16, "p16")
    o = ops.block_matmul_pv(p16, V_, causal=tri)
    assert_parity(host(o), wo, "o")
    ld, lds = H * Dh, H * S
    dv = torch.empty_like(V_); dp = torch.empty_like(s16)
    dq = torch.empty_like(Q); dk = torch.empty_like(Q)
    t1, t2, t3 = (1, 2, 3) if tri else (0, 0, 0)
    ops.gemm_strided_batched(True, False, H, S, Dh, S, 1.0, p16, lds, S, DO, ld, Dh, 0.0, dv, ld, Dh, t3)
    ops.gemm_strided_batched(False, True, H, S, S, Dh, 1.0, DO, ld, Dh, V_, ld, Dh, 0.0, dp, lds, S, t1)
    ds = ops.causal_softmax_bwd(s16, dp)
    ops.gemm_strided_batched(True, False, H, S, Dh, S, alpha, ds, lds, S, Q, ld, Dh, 0.0, dk, ld, Dh, t3)
    ops.gemm_strided_batched(False, False, H, S, Dh, S, alpha, ds, lds, S, K_, ld, Dh, 0.0, dq, ld, Dh, t2)
    assert_parity(host(dv), dv_, "dv")
    assert_parity(host(dq), dq_, "dq")
    assert_parity(host(dk), dk_, "dk")


@pytest.mark.parametrize("S,H,Dh", [(128, 4, 64), (256, 3, 100), (200, 2, 100), (72, 2, 128), (1024, 2, 100),
                                    (384, 6, 100), (8, 1, 4), (192, 4, 60), (130, 2, 124), (448, 2, 100)])
def test_fused_attention(ops, oracle, S, H, Dh):
    """The fused forward and adjoint kernels against the oracle's chain of separate thunks: O, the row
    statistics they keep (maximum and sum of exp of the f16 scores), dQ, dK, dV; ragged sequence lengths
    (rows and keys beyond S are masked) and head dims 4 .. 128; accumulation into existing gradients.
    Both ways of loading tiles are covered: straight into LDS (even head counts with Dh % 8 = 4: every other
    head addressed 4 elements before its start, windows of 8, 13 and 16 chunks; Dh % 8 = 0) and through
    registers (3 heads of 100, 1 head of 4); 448 rows give the dK, dV kernel whole tiles past the diagonal,
    which run as its in-wave pipeline, and a last tile."""
    say("fused attention", S, H, Dh)
    r = rng(1200 + S + Dh)
    alpha = float(np.float32(1.0) / np.sqrt(np.float32(Dh)))
    q, k, v, dO = (randn16(r, (S, H, Dh)) for _ in range(4))
    ws16, wp16, wo = oracle.attention_fwd(q, k, v, alpha)
    dq_, dk_, dv_ = oracle.attention_bwd(q, k, v, dO, alpha)
    Q, K_, V_, DO = dev(q), dev(k), dev(v), dev(dO)
    o, stats = ops.attention_fwd(Q, K_, V_, alpha)
    assert_parity(host(o), wo, "o")
    st = host(stats).reshape(2, H, S)
    low = np.arange(S)[:, None, None] >= np.arange(S)[None, None, :]
    sm = np.where(low, ws16.astype(np.float32), -np.inf)                      # [S, H, S]
    want_m = sm.max(2).T
    want_l = np.exp(sm.astype(np.float64) - sm.max(2, keepdims=True)).sum(2).T
    # up to the few scores whose f16 rounding falls the other way with another fp32 summation order
    assert np.abs(st[0] - want_m).max() <= 2e-3 * max(1.0, np.abs(want_m).max()), "row maxima of the f16 scores"
    assert np.mean(st[0] == want_m) > 0.95
    assert np.abs(st[1] / want_l - 1).max() < 2e-3
    dq, dk, dv = ops.attention_bwd(Q, K_, V_, DO, stats, alpha)
    for name, got, want in (("dv", dv, dv_), ("dq", dq, dq_), ("dk", dk, dk_)):
        assert_parity(host(got), want, name)
    # with the forward output handed over, blocks of queries with spread probabilities take their row sums from
    # dO . O instead of a pass over the keys: the same bar; dV does not depend on the row sums at all
    dq_o, dk_o, dv_o = ops.attention_bwd(Q, K_, V_, DO, stats, alpha, o=o)
    for name, got, want in (("dv", dv_o, dv_), ("dq", dq_o, dq_), ("dk", dk_o, dk_)):
        e2, em = assert_parity(host(got), want, name + " (row sums from dO . O)")
        say("  %s with o: rel_l2 %.2e max_rel %.2e" % (name, e2, em))
    assert_bits(host(dv_o), host(dv), "dv with and without o")
    if S <= 128:                                    # a single block of queries holds row 0: always the pass
        assert_bits(host(dq_o), host(dq), "dq: the first block of queries keeps the pass over the keys")
    # accumulate mode: the product is added to what the tensors hold, one rounding
    base = [randn16(r, (S, H, Dh)) for _ in range(3)]
    acc = tuple(dev(b) for b in base)
    ops.attention_bwd(Q, K_, V_, DO, stats, alpha, acc=acc)
    for name, got, b, plain in zip(("dq", "dk", "dv"), acc, base, (dq, dk, dv)):
        want = b.astype(np.float32) + host(plain).astype(np.float32)
        assert_parity(host(got), want, name + " accumulated", l2=6e-4, mx=2e-3)
    # a second call gives the same bits (no atomics, no order dependence)
    dq2, dk2, dv2 = ops.attention_bwd(Q, K_, V_, DO, stats, alpha)
    for a, b in ((dq, dq2), (dk, dk2), (dv, dv2)):
        assert_bits(host(a), host(b), "repeat")


@pytest.mark.gpu
@pytest.mark.parametrize("gain,exact", [(8.0, False), (24.0, True), (2.0, True)])
def test_fused_attention_with_large_scores(ops, oracle, gain, exact):
    """Scores of large magnitude (row maxima in the hundreds for gain 8, 1500 .. 2600 for 24): by default
    the fused kernels fold the row maximum and the logarithm of the row sum into one fp32 exponent offset,
    whose rounding error is common to a row and grows with |m|; the probabilities are nearly one-hot here,
    the case in which the adjoint's dP - sigma cancels exactly in the reference.  The default forms hold
    the literal bar at gain 8; at gain 24 they do not (dQ 7e-3) and cacti_hip_attention_set_exact(1)
    selects the exactly rounded forms, which do -- they are also run once on ordinary scores."""
    from cacti_amd import ffi
    ffi.call("cacti_hip_attention_set_exact", int(exact))
    try:
        _large_scores_case(ops, oracle, gain)
    finally:
        ffi.call("cacti_hip_attention_set_exact", 0)


def _large_scores_case(ops, oracle, gain):
    S, H, Dh = 384, 3, 100
    say("fused attention, large scores, gain", gain)
    r = rng(1300 + int(gain))
    alpha = float(np.float32(1.0) / np.sqrt(np.float32(Dh)))
    q, k = (randn16(r, (S, H, Dh), gain) for _ in range(2))
    v, dO = (randn16(r, (S, H, Dh)) for _ in range(2))
    ws16, _, wo = oracle.attention_fwd(q, k, v, alpha)
    low = np.arange(S)[:, None, None] >= np.arange(S)[None, None, :]
    m = np.where(low, ws16.astype(np.float32), -np.inf).max(2)
    say("  row maxima of the scores: median %.0f, largest %.0f" % (np.median(np.abs(m)), np.abs(m).max()))
    assert np.abs(m).max() > 9 * gain and np.all(np.isfinite(ws16.astype(np.float32)))
    dq_, dk_, dv_ = oracle.attention_bwd(q, k, v, dO, alpha)
    Q, K_, V_, DO = dev(q), dev(k), dev(v), dev(dO)
    o, stats = ops.attention_fwd(Q, K_, V_, alpha)
    e2, em = assert_parity(host(o), wo, "o")
    say("  o  rel_l2 %.2e max_rel %.2e" % (e2, em))
    # the forward output is handed over: rows this concentrated must all fall back to the pass over the keys
    dq, dk, dv = ops.attention_bwd(Q, K_, V_, DO, stats, alpha, o=o)
    for name, got, want in (("dv", dv, dv_), ("dq", dq, dq_), ("dk", dk, dk_)):
        e2, em = assert_parity(host(got), want, name)
        say("  %s rel_l2 %.2e max_rel %.2e" % (name, e2, em))


@pytest.mark.gpu
@pytest.mark.parametrize("S,H,Dh", [(64, 4, 64), (2048, 32, 100), (37, 4, 20), (16, 4, 6)])
def test_rope_on_two_tensors_in_one_launch(S, H, Dh):
    """cacti_hip_rope_{fwd,bwd}_pair: bit for bit what two single launches give, accumulation included
    (Dh = 6 takes the staged kernel, one launch per tensor behind the same entry point)."""
    import torch
    from cacti_amd import ffi, ops
    g = torch.Generator(device="cuda").manual_seed(S + Dh)
    x0, x1, a0, a1 = (torch.randn(S, H, Dh, device="cuda", generator=g).half() for _ in range(4))
    cos, sin = ops.rope_tables(S, Dh)
    st = torch.cuda.current_stream().cuda_stream
    y0, y1 = torch.empty_like(x0), torch.empty_like(x1)
    ffi.call("cacti_hip_rope_fwd_pair", S, H, Dh, x0.data_ptr(), x1.data_ptr(), cos.data_ptr(), sin.data_ptr(),
             y0.data_ptr(), y1.data_ptr(), st)
    assert torch.equal(y0, ops.rope_fwd(x0, cos, sin)) and torch.equal(y1, ops.rope_fwd(x1, cos, sin))
    d0, d1 = a0.clone(), torch.empty_like(x1)
    ffi.call("cacti_hip_rope_bwd_pair", S, H, Dh, x0.data_ptr(), x1.data_ptr(), cos.data_ptr(), sin.data_ptr(),
             d0.data_ptr(), 1, d1.data_ptr(), 0, st)
    w0 = a0.clone()
    ffi.call("cacti_hip_rope_bwd", S, H, Dh, x0.data_ptr(), cos.data_ptr(), sin.data_ptr(), w0.data_ptr(), 1, st)
    assert torch.equal(d0, w0) and torch.equal(d1, ops.rope_bwd(x1, cos, sin))
