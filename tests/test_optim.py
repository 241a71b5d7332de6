"""AdamW32 optimiser thunks (src/librarium/adamw.rs:45-60; OnlineAverageScale, OnlineAverageSquareScale,
OnlineAdamWUpdate, src/thunk/op.rs:3884-4062; the driver's host arithmetic, src/op.rs:984-1023; the cast
of the master weights back to f16, src/op.rs:1112-1135).

CPU: the oracle's restatement against torch.optim.AdamW in float64 (an independent implementation of
the same update: betas = 1 - a, bias corrections folded differently), closed forms of the moving
averages and special cases that isolate every term.  GPU: the HIP kernels, one thunk at a time and the
one-launch step over a list of tensors, against the oracle bit for bit (every operation is a correctly
rounded f32 add, multiply, divide or square root on both sides, in the same order)."""
import numpy as np
import pytest

from tests.util import rng

OPT = dict(grad_scale=1024.0, lr=2.0e-5, wd=0.1, a1=0.1, a2=0.05, eps=1.0e-5)     # open_llama_3b_train.rs:47-54


@pytest.fixture(scope="module")
def ops():
    import torch
    assert torch.cuda.is_available(), "these tests need the MI355X"
    from cacti_amd import ops as o
    return o


# ------------------------------------------------------------------------------------------ oracle
def test_oracle_scalars_follow_the_closed_forms(oracle):
    for it in (1, 2, 3, 7, 100, 5000):
        s = oracle.adamw32_scalars(it, **OPT).astype(np.float64)
        a1, a2 = np.float64(np.float32(OPT["a1"])), np.float64(np.float32(OPT["a2"]))
        u1, u2 = 1 - (1 - a1) ** it, np.sqrt(1 - (1 - a2) ** it)
        want = [1 / 1024.0, a1, a2, -np.float64(np.float32(OPT["lr"])), u2 / u1, np.float64(np.float32(OPT["wd"])),
                np.float64(np.float32(OPT["eps"])) * u2]
        assert np.allclose(s, want, rtol=2e-6, atol=0), (it, s, want)
    # first iteration: the reference takes a1 and sqrt(a2) themselves, not 1 - (1 - a)
    s = oracle.adamw32_scalars(1, **OPT)
    assert s[4] == np.sqrt(np.float32(OPT["a2"])) / np.float32(OPT["a1"])
    assert s[6] == np.float32(OPT["eps"]) * np.sqrt(np.float32(OPT["a2"]))
    assert s[0] == np.float32(1.0 / 1024.0) and s[3] == -np.float32(OPT["lr"])
    assert oracle.adamw32_scalars(3, **dict(OPT, grad_scale=None))[0] == 1.0
    for bad in (0, -1):
        with pytest.raises(ValueError):
            oracle.adamw32_scalars(bad, **OPT)


def test_oracle_moving_averages_closed_forms(oracle):
    r = rng(1)
    u = (r.standard_normal(4099) * 3).astype(np.float16)
    uf = u.astype(np.float64)
    v0 = r.standard_normal(4099).astype(np.float32)
    # rate 0 keeps v, rate 1 replaces it (up to the rounding of (x - v) + v)
    assert np.array_equal(oracle.online_average_scale(u, v0, 0.25, 0.0), v0)
    assert np.array_equal(oracle.online_average_square_scale(u, v0, 0.25, 0.0), v0)
    assert np.allclose(oracle.online_average_scale(u, v0, 0.25, 1.0), 0.25 * uf, rtol=0, atol=2e-7 * 8)
    assert np.allclose(oracle.online_average_square_scale(u, v0, 0.25, 1.0), (0.25 * uf) ** 2, rtol=0, atol=1e-6)
    # the scale is applied to u before squaring: (s u)^2, not s u^2
    one = oracle.online_average_square_scale(np.float16([2.0]), np.float32([0.0]), 0.5, 1.0)
    assert one[0] == 1.0
    # k steps from v0 with a constant source: v_k = x + (1 - rate)^k (v0 - x)
    for fn, x in ((oracle.online_average_scale, 0.5 * uf), (oracle.online_average_square_scale, (0.5 * uf) ** 2)):
        v = v0
        for _ in range(9):
            v = fn(u, v, 0.5, 0.125)
        want = x + (1 - 0.125) ** 9 * (v0.astype(np.float64) - x)
        assert np.allclose(v, want, rtol=2e-6, atol=2e-6)


def test_oracle_update_special_cases(oracle):
    r = rng(2)
    n = 1000
    g1 = r.standard_normal(n).astype(np.float32)
    g2 = (r.standard_normal(n) ** 2).astype(np.float32)
    w = r.standard_normal(n).astype(np.float32)
    z = np.zeros(n, np.float32)
    # no gradient, no decay: unchanged; decay alone: w (1 + slr lam); sign: the step goes against g1
    assert np.array_equal(oracle.online_adamw_update(z, g2, w, -0.1, 2.0, 0.0, 1e-3), w)
    assert np.allclose(oracle.online_adamw_update(z, g2, w, -0.1, 2.0, 0.5, 1e-3), w.astype(np.float64) * (1 - 0.05),
                       rtol=3e-7, atol=0)
    d = oracle.online_adamw_update(g1, g2, z, -0.1, 2.0, 0.0, 1e-3)
    assert np.all(np.sign(d) == -np.sign(g1))
    # v = 0: the step is slr lru u / eps (eps is added to the root, not put under it)
    assert np.allclose(oracle.online_adamw_update(g1, z, z, -0.1, 2.0, 0.0, 1e-3), -0.1 * 2.0 * g1.astype(np.float64) / 1e-3,
                       rtol=3e-7, atol=0)
    want = w.astype(np.float64) - 0.1 * (2.0 * g1.astype(np.float64) / (np.sqrt(g2.astype(np.float64)) + 1e-3) + 0.5 * w)
    assert np.allclose(oracle.online_adamw_update(g1, g2, w, -0.1, 2.0, 0.5, 1e-3), want, rtol=2e-6, atol=1e-6)


def test_oracle_adamw32_matches_torch_adamw_in_float64(oracle):
    """Six steps of three tensors against torch.optim.AdamW (float64): same update, written with
    betas and separate bias corrections.  The gradients are f16 and scaled by 1024 as in the example."""
    import torch
    r = rng(3)
    shapes = [(37, 53), (64,), (5, 7, 3)]
    w0 = [(r.standard_normal(s) * 0.05).astype(np.float16) for s in shapes]
    tw = [torch.tensor(w.astype(np.float64), requires_grad=True) for w in w0]
    topt = torch.optim.AdamW(tw, lr=float(np.float32(OPT["lr"])) * 50, betas=(1 - float(np.float32(OPT["a1"])), 1 - float(np.float32(OPT["a2"]))),
                             eps=float(np.float32(OPT["eps"])), weight_decay=float(np.float32(OPT["wd"])))
    opt = dict(OPT, lr=OPT["lr"] * 50)                       # a larger rate, so a wrong step shows
    master = [w.astype(np.float32) for w in w0]              # set_cast
    avg = [np.zeros(s, np.float32) for s in shapes]
    avg2 = [np.zeros(s, np.float32) for s in shapes]
    for it in range(1, 7):
        sc = oracle.adamw32_scalars(it, **opt)
        grads = [(r.standard_normal(s) * 0.3 * (1 + it % 3)).astype(np.float16) for s in shapes]
        for k in range(3):
            tw[k].grad = torch.tensor(grads[k].astype(np.float64) / 1024.0)
            avg[k], avg2[k], master[k], p16 = oracle.adamw32_step(grads[k], avg[k], avg2[k], master[k], sc)
            assert np.array_equal(p16.view(np.uint16), master[k].astype(np.float16).view(np.uint16))
        topt.step()
        for k in range(3):
            want = tw[k].detach().numpy()
            err = np.abs(master[k] - want).max() / np.abs(want).max()
            assert err < 2e-6, (it, k, err)
    # the parameters moved by far more than the agreement asked for
    assert np.abs(master[0] - w0[0].astype(np.float32)).max() > 1e-3


def test_oracle_step_is_the_four_thunks_in_order(oracle):
    r = rng(4)
    g = (r.standard_normal(1001) * 0.5).astype(np.float16)
    a, b, w = (r.standard_normal(1001).astype(np.float32) for _ in range(3))
    b = b * b
    sc = oracle.adamw32_scalars(4, **OPT)
    a1, b1, w1, p1 = oracle.adamw32_step(g, a, b, w, sc)
    a2 = oracle.online_average_scale(g, a, sc[0], sc[1])
    b2 = oracle.online_average_square_scale(g, b, sc[0], sc[2])
    w2 = oracle.online_adamw_update(a2, b2, w, sc[3], sc[4], sc[5], sc[6])
    assert np.array_equal(a1, a2) and np.array_equal(b1, b2) and np.array_equal(w1, w2)
    assert np.array_equal(p1.view(np.uint16), oracle.cast_f32_f16(w2).view(np.uint16))


# ------------------------------------------------------------------------------------------ GPU
def _bits(x):
    return np.ascontiguousarray(x).view(np.uint16 if x.dtype == np.float16 else np.uint32)


def _t(x):
    import torch
    return torch.from_numpy(np.ascontiguousarray(x)).cuda()


def _state(r, n, kind):
    g = (r.standard_normal(n) * (1e-4 if kind == "tiny" else 0.5) * 1024).astype(np.float16)
    if kind == "zeros":
        g[r.random(n) < 0.5] = 0
    a = (r.standard_normal(n) * 1e-3).astype(np.float32)
    b = ((r.standard_normal(n) * 1e-3) ** 2).astype(np.float32)
    if kind == "zeros":
        a[::3] = 0
        b[::2] = 0
    w = (r.standard_normal(n) * 0.05).astype(np.float32)
    return g, a, b, w


SIZES = [0, 1, 7, 8, 9, 1000, 8192, 8192 * 3 + 5, 1 << 20]


@pytest.mark.gpu
@pytest.mark.parametrize("n", SIZES)
def test_thunks_match_the_oracle_bit_for_bit(ops, oracle, n):
    r = rng(100 + n % 97)
    for kind in ("plain", "tiny", "zeros"):
        print("optim thunks", n, kind, flush=True)
        g, a, b, w = _state(r, n, kind)
        sc = oracle.adamw32_scalars(3, **OPT)
        ga = ops.online_average_scale_(_t(g), _t(a), float(sc[0]), float(sc[1])).cpu().numpy()
        gb = ops.online_average_square_scale_(_t(g), _t(b), float(sc[0]), float(sc[2])).cpu().numpy()
        gw = ops.online_adamw_update_(_t(a), _t(b), _t(w), *[float(x) for x in sc[3:7]]).cpu().numpy()
        assert np.array_equal(_bits(ga), _bits(oracle.online_average_scale(g, a, sc[0], sc[1])))
        assert np.array_equal(_bits(gb), _bits(oracle.online_average_square_scale(g, b, sc[0], sc[2])))
        assert np.array_equal(_bits(gw), _bits(oracle.online_adamw_update(a, b, w, *sc[3:7])))
        assert np.array_equal(_bits(ops.cast_f32_f16(_t(w)).cpu().numpy()), _bits(oracle.cast_f32_f16(w)))
        assert np.array_equal(_bits(ops.cast_f16_f32(_t(g)).cpu().numpy()), _bits(g.astype(np.float32)))


@pytest.mark.gpu
def test_casts_cover_every_f16_pattern_and_the_rounding_boundaries(ops, oracle):
    allh = np.arange(65536, dtype=np.uint32).astype(np.uint16).view(np.float16)
    up = ops.cast_f16_f32(_t(allh)).cpu().numpy()
    fin = np.isfinite(allh)
    assert np.array_equal(_bits(up[fin]), _bits(allh[fin].astype(np.float32)))
    assert np.array_equal(np.isnan(up), np.isnan(allh)) and np.array_equal(np.isinf(up), np.isinf(allh))
    # f32 -> f16: every f16 value, the midpoints between neighbours and their f32 neighbours
    # (ties to even, overflow to inf at 65520, subnormal results)
    h32 = allh[fin].astype(np.float32)
    with np.errstate(over="ignore"):
        nxt = np.nextafter(allh[fin], np.float16(np.inf)).astype(np.float32)
    mid = ((h32.astype(np.float64) + nxt.astype(np.float64)) / 2).astype(np.float32)
    x = np.concatenate([h32, mid, np.nextafter(mid, np.float32(np.inf)), np.nextafter(mid, np.float32(-np.inf)),
                        np.float32([65519.99, 65520.0, 1e30, -1e30, 2.0 ** -25, 2.0 ** -25 * 1.0001, 1e-30])])
    x = x[np.isfinite(x)]
    got = ops.cast_f32_f16(_t(x)).cpu().numpy()
    assert np.array_equal(_bits(got), _bits(oracle.cast_f32_f16(x)))
    with np.errstate(over="ignore"):
        assert np.array_equal(_bits(got), _bits(x.astype(np.float16)))


@pytest.mark.gpu
def test_one_launch_step_matches_the_oracle_over_three_iterations(ops, oracle):
    """Ragged list of tensors (an empty one, sizes not divisible by 8, several workgroups), three
    steps with new gradients each: averages, master weights and f16 parameters bit-exact."""
    import torch
    r = rng(9)
    ns = [7, 8192 * 2 + 3, 0, 1, 4096, 100003, 8]
    kinds = ["plain", "tiny", "plain", "zeros", "zeros", "plain", "tiny"]
    st = [_state(r, n, k) for n, k in zip(ns, kinds)]
    a = [s[1] for s in st]; b = [s[2] for s in st]; w = [s[3] for s in st]
    da, db, dw = [_t(x) for x in a], [_t(x) for x in b], [_t(x) for x in w]
    dp = [torch.empty(n, dtype=torch.float16, device="cuda") for n in ns]
    for it in (1, 2, 3):
        print("optim batch iteration", it, flush=True)
        sc = oracle.adamw32_scalars(it, **OPT)
        gsc = ops.adamw32_scalars(it, **OPT)
        assert np.array_equal(np.float32(gsc), sc)
        g = [_state(r, n, k)[0] for n, k in zip(ns, kinds)]
        ops.adamw32_step_([_t(x) for x in g], da, db, dw, dp, gsc)
        for k in range(len(ns)):
            a[k], b[k], w[k], p = oracle.adamw32_step(g[k], a[k], b[k], w[k], sc)
            assert np.array_equal(_bits(da[k].cpu().numpy()), _bits(a[k])), (it, k)
            assert np.array_equal(_bits(db[k].cpu().numpy()), _bits(b[k])), (it, k)
            assert np.array_equal(_bits(dw[k].cpu().numpy()), _bits(w[k])), (it, k)
            assert np.array_equal(_bits(dp[k].cpu().numpy()), _bits(p)), (it, k)


@pytest.mark.gpu
def test_scalars_reject_a_non_positive_iteration(ops):
    from cacti_amd.ffi import CactiError
    for bad in (0, -3):
        with pytest.raises(CactiError) as e:
            ops.adamw32_scalars(bad, **OPT)
        assert e.value.code == -1 and "iter_nr" in str(e.value)


@pytest.mark.gpu
def test_non_finite_gradients_propagate(ops, oracle):
    """inf / nan in the gradient reach the averages, the master weights and the parameters as
    non-finite values in the same places as in the oracle (payloads aside)."""
    import torch
    r = rng(12)
    g, a, b, w = _state(r, 4099, "plain")
    g[5] = np.float16("inf"); g[77] = np.float16("nan"); g[4098] = -np.float16("inf")
    sc = oracle.adamw32_scalars(2, **OPT)
    da, db, dw, dp = _t(a), _t(b), _t(w), torch.empty(4099, dtype=torch.float16, device="cuda")
    ops.adamw32_step_([_t(g)], [da], [db], [dw], [dp], [float(x) for x in sc])
    oa, ob, ow, op_ = oracle.adamw32_step(g, a, b, w, sc)
    for got, want in ((da, oa), (db, ob), (dw, ow), (dp, op_)):
        got = got.cpu().numpy()
        assert np.array_equal(np.isnan(got), np.isnan(want)) and np.array_equal(np.isinf(got), np.isinf(want))
        ok = np.isfinite(want)
        assert np.array_equal(_bits(got[ok]), _bits(want[ok]))
