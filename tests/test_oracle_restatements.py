"""Pins the oracle's restatement modes (no GPU needed).

The composed-cycle tests hold the device to the spread of twelve restatements of the oracle
(tests/envelope.py).  That bar means something only if every restatement is itself a correct
statement of the same arithmetic and the set cannot grow unnoticed, so:

  * the set is frozen: RESTATEMENTS must equal the literal below, GEMM_ORDERS likewise;
  * every GEMM order is checked against fp64 arithmetic: exact on integer-valued operands (any
    summation order of exactly representable partial sums gives the same fp32 value, so a dropped,
    doubled or misplaced k fails), and on random operands within half an f16 ulp + fp32 noise with
    >= 99 % of the f16 results bit-identical to the rounded fp64 product, for all four transposes;
  * the orders really differ (else the envelope would measure nothing): on a long ill-conditioned sum
    at least 7 of the 8 give pairwise different fp32 results;
  * reduce_f32 / exp_exact: softmax, cross-entropy and the RMSNorm under each switch against scipy /
    numpy fp64 closed forms, at fp32-level tolerances per call, and one switch moves a result by no
    more than a few fp32 ulps.
"""
import itertools

import numpy as np
import pytest
import scipy.special as sp

from tests.util import f64, rel_l2, rng, randn16

FROZEN_ORDERS = {"ascending": (0, 0, 0), "descending": (0, 1, 0), "blocked64": (64, 0, 0), "pairwise": (32, 0, 1),
                 "blocked16": (16, 0, 0), "blocked64rev": (64, 1, 0), "pairwise8": (8, 0, 1),
                 "blocked256": (256, 0, 0)}
FROZEN_RESTATEMENTS = {
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


@pytest.fixture()
def restore(oracle):
    yield oracle
    oracle.set_restatement("ascending")


def test_the_set_of_restatements_is_frozen(oracle):
    """The envelope is a maximum over pairs of these runs and grows with every member: adding one is a
    change of the parity bar and has to be made here, in the open."""
    assert dict(oracle.GEMM_ORDERS) == FROZEN_ORDERS
    assert dict(oracle.RESTATEMENTS) == FROZEN_RESTATEMENTS
    assert list(oracle.RESTATEMENTS)[0] == "ascending"          # the default run every test compares with


def _operands(r, ta, tb, M, N, K, integer):
    def draw(shape):
        if integer:
            return r.integers(-8, 9, shape).astype(np.float16)
        return randn16(r, shape)
    A = draw((K, M) if ta else (M, K))
    B = draw((N, K) if tb else (K, N))
    return A, B, (f64(A).T if ta else f64(A)), (f64(B).T if tb else f64(B))


@pytest.mark.parametrize("order", list(FROZEN_ORDERS))
def test_every_gemm_order_is_exact_on_integers(restore, order):
    """Integers in [-8, 8]: every partial sum is an integer below 2^24, exact in fp32 whatever the order,
    and the results (|c| <= 64 K) are kept below the f16 rounding grain by K <= 31, so C must equal the
    fp64 product exactly; a second, longer case checks the fp32 sum before the rounding through alpha."""
    o = restore
    o.set_gemm_order(order)
    r = rng(77)
    for ta, tb in itertools.product((0, 1), repeat=2):
        A, B, opA, opB = _operands(r, ta, tb, 19, 23, 31, True)
        got = o.matmul(ta, tb, A, B)
        assert np.array_equal(f64(got), opA @ opB), (order, ta, tb)
    # K = 1000 (ragged against every run length 8 .. 256): |sum| <= 64000 < 2^24 exact in fp32; alpha = 2^-6
    # brings it to <= 1000 where f16 keeps multiples of 1/2 — the expected value is the rounded exact one
    A, B, opA, opB = _operands(r, 0, 1, 37, 29, 1000, True)
    got = o.matmul(0, 1, A, B, alpha=2.0 ** -6)
    want = ((opA @ opB) * 2.0 ** -6).astype(np.float16)
    assert np.array_equal(got.view(np.uint16), want.view(np.uint16)), order


@pytest.mark.parametrize("order", list(FROZEN_ORDERS))
def test_every_gemm_order_against_fp64(restore, order):
    """37 x 29 x 1000, N(0, 1) operands, all four transposes, with alpha and beta: each element within half
    an f16 ulp of the fp64 value plus the fp32 accumulation noise, and >= 99 % of the f16 results the very
    bits of the rounded fp64 product."""
    o = restore
    o.set_gemm_order(order)
    r = rng(78)
    for ta, tb in itertools.product((0, 1), repeat=2):
        A, B, opA, opB = _operands(r, ta, tb, 37, 29, 1000, False)
        C0 = randn16(r, (37, 29))
        for alpha, beta in ((1.0, 0.0), (0.1, 1.0)):
            got = o.matmul(ta, tb, A, B, alpha, beta, C0)
            want = alpha * (opA @ opB) + beta * f64(C0)
            assert np.all(np.abs(f64(got) - want) <= 2.0 ** -11 * np.abs(want) + 2e-4), (order, ta, tb)
            same = np.mean(got.view(np.uint16) == want.astype(np.float16).view(np.uint16))
            assert same >= 0.99, (order, ta, tb, alpha, same)


def test_the_gemm_orders_are_different_sums(restore):
    """64 x 64 dot products of 4096 terms of widely mixed magnitude (log-normal factors), where the fp32
    differences between summation orders reach the f16 result now and then: at least 7 of the 8 orders must
    give a result matrix different from every other one, and each is the same product to rounding."""
    o = restore
    r = rng(79)
    K = 4096
    A = (0.05 * r.standard_normal((64, K)) * np.exp(r.standard_normal((64, K)) * 2)).astype(np.float16)
    B = (0.05 * r.standard_normal((64, K)) * np.exp(r.standard_normal((64, K)) * 2)).astype(np.float16)
    outs = {}
    for order in FROZEN_ORDERS:
        o.set_gemm_order(order)
        outs[order] = o.matmul(0, 1, A, B).tobytes()
    assert len(set(outs.values())) >= 7, "the orders collapse to %d distinct results" % len(set(outs.values()))
    # and all of them are the same product to rounding
    ref = f64(A) @ f64(B).T
    for order in FROZEN_ORDERS:
        got = np.frombuffer(outs[order], np.float16).reshape(64, 64)
        assert rel_l2(got, ref) < 1e-3, order


SWITCHES = [(0, 0), (1, 0), (0, 1), (1, 1)]


@pytest.mark.parametrize("red,ex", SWITCHES)
def test_softmax_and_cross_entropy_under_each_switch(restore, red, ex):
    """Causal softmax, its adjoint, the cross-entropy loss and its adjoint with reductions in f32 / f64 and
    exp / log from libm / correctly rounded: each against scipy's fp64 closed forms at the tolerance one
    f16 (or, for the f32 loss, a few f32) roundings allow."""
    o = restore
    o.set_reduce_f32(red)
    o.set_exp_exact(ex)
    r = rng(80)
    S, H = 48, 3
    s16 = randn16(r, (S, H, S), 2.0)
    low = np.arange(S)[:, None, None] >= np.arange(S)[None, None, :]
    masked = np.where(low, f64(s16), -np.inf)
    p = sp.softmax(masked, axis=2)
    got = o.causal_softmax_fwd(s16)
    assert np.all(np.abs(f64(got) - p) <= 2.0 ** -11 * p + 1e-7), (red, ex)
    assert np.all(f64(got)[~np.broadcast_to(low, got.shape)] == 0)
    dp16 = randn16(r, (S, H, S))
    t = p * f64(dp16)
    ds = np.where(low, t - p * t.sum(2, keepdims=True), 0.0)
    gds = o.causal_softmax_bwd(s16, dp16)
    assert np.all(np.abs(f64(gds) - ds) <= 2.0 ** -10 * np.abs(ds) + 3e-6), (red, ex)

    N, V = 40, 1000
    logit = randn16(r, (N, V), 3.0)
    tok = r.integers(0, V, N).astype(np.uint16)
    scale = (r.random(N) + 0.5).astype(np.float32)
    _, loss, amax = o.softmax_ce_fwd(logit, tok, want_prob=False)
    lse = sp.logsumexp(f64(logit), axis=1)
    want_loss = lse - f64(logit)[np.arange(N), tok]
    assert np.all(np.abs(f64(loss) - want_loss) <= 4e-6 * np.maximum(1.0, np.abs(want_loss))), (red, ex)
    assert np.array_equal(amax, np.argmax(f64(logit), axis=1).astype(np.uint16))
    dl = o.softmax_ce_bwd(logit, tok, scale)
    z = sp.softmax(f64(logit), axis=1)
    z[np.arange(N), tok] -= 1.0
    want_dl = z * f64(scale)[:, None]
    assert np.all(np.abs(f64(dl) - want_dl) <= 2.0 ** -10 * np.abs(want_dl) + 1e-7), (red, ex)


@pytest.mark.parametrize("red,ex", SWITCHES)
def test_rmsnorm_under_each_switch(restore, red, ex):
    """The RMSNorm row reduction (and the adjoint's two) in f32 or f64: forward against the closed form,
    adjoint against the closed forms `dx = (g - t mean(g t)) / r` with g = dy w, and `dw = sum_n dy t`."""
    o = restore
    o.set_reduce_f32(red)
    o.set_exp_exact(ex)
    r = rng(81)
    N, D = 33, 320
    x, w, dy = randn16(r, (N, D)), randn16(r, (D,)), randn16(r, (N, D))
    eps = 1e-6
    y, _, _ = o.rmsnorm_fwd(x, w, eps)
    rr = np.sqrt((f64(x) ** 2).mean(1, keepdims=True) + eps)
    t = f64(x) / rr
    assert np.all(np.abs(f64(y) - f64(w) * t) <= 2.0 ** -11 * np.abs(f64(w) * t) + 1e-6)
    dx, dw = o.rmsnorm_bwd(x, w, eps, dy)
    g = f64(dy) * f64(w)
    want_dx = (g - t * (g * t).mean(1, keepdims=True)) / rr
    assert rel_l2(dx, want_dx) < 6e-4            # two f16 contributions added in f16
    assert rel_l2(dw, (f64(dy) * t).sum(0)) < 6e-4


def test_a_switch_moves_a_result_by_ulps_only(restore):
    """reduce_f32 and exp_exact change the f32 loss of a row by a few f32 ulps, never more: they are
    restatements of the same arithmetic, not different arithmetic."""
    o = restore
    r = rng(82)
    N, V = 64, 4000
    logit = randn16(r, (N, V), 3.0)
    tok = r.integers(0, V, N).astype(np.uint16)
    losses = {}
    for red, ex in SWITCHES:
        o.set_reduce_f32(red)
        o.set_exp_exact(ex)
        losses[(red, ex)] = o.softmax_ce_fwd(logit, tok, want_prob=False)[1].astype(np.float32)
    base = losses[(0, 0)]
    for key, l in losses.items():
        ulps = np.abs(l.view(np.int32).astype(np.int64) - base.view(np.int32).astype(np.int64))
        assert ulps.max() <= 16, (key, int(ulps.max()))
    assert any(not np.array_equal(l, base) for l in losses.values())      # and they are not no-ops
