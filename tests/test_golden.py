"""Committed fixtures (tests/golden/*.npz, written by tests/golden/make_fixtures.py).

CPU: the oracle still produces them (guards the checker itself against drift).
GPU: the HIP path, called through the C ABI, reproduces them to the parity bar of
tests/util.py (rel-L2 <= 1e-3, max element relative error <= 2e-2; indices bit-exact).
"""
import importlib.util
import os

import numpy as np
import pytest

from tests.util import assert_parity

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
# genuine uint16 (token ids, bf16 bit patterns); any other uint16 array holds f16 bits
INTS = {"in_tok", "in_idx", "in_lm_tok", "out_amax", "out_tok", "in_bf16", "out_f32_bf16", "out_f16_bf16"}
UNITS = ["rmsnorm", "rope_dh12", "rope_dh100", "silu_gate", "causal_softmax", "softmax_ce", "embed",
         "matmul", "attention", "llama_tiny", "digests", "optimizer", "raw_casts", "llama_cached_tiny"]
EXACT = {"digests", "optimizer", "raw_casts"}               # integer, byte and f32 element-wise work: every bit


def load(name):
    z = np.load(os.path.join(GOLDEN, name + ".npz"), allow_pickle=False)
    return {k: (z[k].view(np.float16) if z[k].dtype == np.uint16 and k not in INTS else z[k])
            for k in z.files}


def close_enough(got, want, name):
    got = np.asarray(got).reshape(want.shape)
    if want.dtype in (np.uint16, np.int16, np.int32, np.int64):
        assert np.array_equal(got, want), name
    elif want.size == 1:
        assert float(got.ravel()[0]) == float(want.ravel()[0]), name
    else:
        assert_parity(np.asarray(got), want, name)


def test_fixture_files_are_complete():
    for u in UNITS:
        d = load(u)
        assert any(k.startswith("in_") for k in d) and any(k.startswith("out_") for k in d), u


def test_oracle_reproduces_fixtures(oracle):
    """Bit patterns match on the build that wrote them; another CPU's GEMM micro-kernel may sum
    in a different order, so the assertion is the parity bar plus >= 99 % identical f16 bits."""
    spec = importlib.util.spec_from_file_location("make_fixtures", os.path.join(GOLDEN, "make_fixtures.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    fresh = mod.units()
    assert sorted(fresh) == sorted(UNITS)
    for u in UNITS:
        want = load(u)
        assert sorted(want) == sorted(fresh[u]), u
        for k, w in want.items():
            g = np.asarray(fresh[u][k])
            if u in EXACT:
                assert np.ascontiguousarray(g).tobytes() == np.ascontiguousarray(w).tobytes(), (u, k)
                continue
            close_enough(g, w, u + "." + k)
            if w.dtype == np.float16 and w.size >= 64:
                same = np.mean(np.ascontiguousarray(g).view(np.uint16) == np.ascontiguousarray(w).view(np.uint16))
                assert same >= 0.99, (u, k, same)


# ------------------------------------------------------------------ GPU side
def _dev(a):
    import torch
    if a.dtype == np.uint16:
        a = a.view(np.int16)
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _host(t):
    return t.detach().cpu().numpy()


@pytest.fixture(scope="module")
def ops():
    import torch
    assert torch.cuda.is_available(), "these tests need the MI355X"
    from cacti_amd import ops as o
    return o


@pytest.mark.gpu
def test_gpu_adjoint_kernels_hit_fixtures(ops):
    d = load("rmsnorm")
    x, w, dy = _dev(d["in_x"]), _dev(d["in_w"]), _dev(d["in_dy"])
    close_enough(_host(ops.rms_norm_fwd(x, w, 1e-6)), d["out_y"], "rmsnorm.y")
    dx, dw = ops.rms_norm_bwd(x, w, 1e-6, dy)
    close_enough(_host(dx), d["out_dx"], "rmsnorm.dx")
    close_enough(_host(dw), d["out_dw"], "rmsnorm.dw")
    dx, dw = ops.rms_norm_bwd(x, w, 1e-6, dy, _dev(d["in_dx0"]), _dev(d["in_dw0"]))
    close_enough(_host(dx), d["out_dx_acc"], "rmsnorm.dx_acc")
    close_enough(_host(dw), d["out_dw_acc"], "rmsnorm.dw_acc")

    for tag in ("rope_dh12", "rope_dh100"):
        d = load(tag)
        S, H, Dh = d["in_x"].shape
        cos, sin = ops.rope_tables(S, Dh)
        close_enough(_host(cos), d["out_cos"], tag + ".cos")
        close_enough(_host(sin), d["out_sin"], tag + ".sin")
        cos, sin = _dev(d["out_cos"]), _dev(d["out_sin"])
        close_enough(_host(ops.rope_fwd(_dev(d["in_x"]), cos, sin)), d["out_y"], tag + ".y")
        close_enough(_host(ops.rope_bwd(_dev(d["in_dy"]), cos, sin)), d["out_dx"], tag + ".dx")
        close_enough(_host(ops.rope_bwd(_dev(d["in_dy"]), cos, sin, _dev(d["in_dx0"]))),
                     d["out_dx_acc"], tag + ".dx_acc")

    d = load("silu_gate")
    g, u, dh = _dev(d["in_g"]), _dev(d["in_u"]), _dev(d["in_dh"])
    close_enough(_host(ops.silu_gate_fwd(g, u)), d["out_h"], "silu.h")
    dg, du = ops.silu_gate_bwd(g, u, dh)
    close_enough(_host(dg), d["out_dg"], "silu.dg")
    close_enough(_host(du), d["out_du"], "silu.du")
    dg, du = ops.silu_gate_bwd(g, u, dh, _dev(d["in_dg0"]), _dev(d["in_du0"]))
    close_enough(_host(dg), d["out_dg_acc"], "silu.dg_acc")
    close_enough(_host(du), d["out_du_acc"], "silu.du_acc")

    d = load("causal_softmax")
    s16 = _dev(d["in_s16"])
    S = d["in_s16"].shape[0]
    low = np.broadcast_to(np.arange(S)[:, None, None] >= np.arange(S)[None, None, :], d["in_s16"].shape)
    close_enough(np.where(low, _host(ops.causal_softmax_fwd(s16)), 0).astype(np.float16), d["out_p16"], "csm.p16")
    close_enough(np.where(low, _host(ops.causal_softmax_bwd(s16, _dev(d["in_dp16"]))), 0).astype(np.float16),
                 d["out_ds16"], "csm.ds16")

    d = load("softmax_ce")
    logit, tok = _dev(d["in_logit"]), _dev(d["in_tok"])
    prob, loss, amax = ops.softmax_ce_fwd(logit, tok)
    close_enough(_host(prob), d["out_prob"], "ce.prob")
    close_enough(_host(loss), d["out_loss"], "ce.loss")
    assert np.array_equal(_host(amax).view(np.uint16), d["out_amax"])
    close_enough(_host(ops.softmax_ce_bwd(logit, tok, _dev(d["in_scale"]))), d["out_dlogit"], "ce.dlogit")

    d = load("embed")
    y = _host(ops.embed_fwd(_dev(d["in_W"]), _dev(d["in_idx"])))
    assert np.array_equal(y.view(np.uint16), d["out_y"].view(np.uint16))            # a gather is exact
    close_enough(_host(ops.embed_bwd(d["in_W"].shape[0], _dev(d["in_idx"]), _dev(d["in_dy"]))),
                 d["out_dW"], "embed.dW")


@pytest.mark.gpu
def test_gpu_gemm_and_attention_hit_fixtures(ops):
    import torch
    d = load("matmul")
    for ta in (0, 1):
        for tb in (0, 1):
            t = "NT"[ta] + "NT"[tb]
            A, B = _dev(d["in_A_" + t]), _dev(d["in_B_" + t])
            close_enough(_host(ops.gemm(A, B, bool(ta), bool(tb))), d["out_C_" + t], "C_" + t)
            c = _dev(d["in_C0"])
            close_enough(_host(ops.gemm(A, B, bool(ta), bool(tb), 0.25, 1.0, c)), d["out_Cacc_" + t],
                         "Cacc_" + t)

    d = load("attention")
    q, k, v, dO = (_dev(d[n]) for n in ("in_q", "in_k", "in_v", "in_dO"))
    S, H, Dh = d["in_q"].shape
    alpha = float(d["in_alpha"].ravel()[0])
    low = np.broadcast_to(np.arange(S)[:, None, None] >= np.arange(S)[None, None, :], d["out_s16"].shape)
    s16 = ops.block_matmul_qk(q, k, alpha, causal=True)
    close_enough(np.where(low, _host(s16), 0).astype(np.float16),
                 np.where(low, d["out_s16"], 0).astype(np.float16), "attn.s16")
    p16 = ops.causal_softmax_fwd(s16)
    close_enough(np.where(low, _host(p16), 0).astype(np.float16), d["out_p16"], "attn.p16")
    close_enough(_host(ops.block_matmul_pv(p16, v, causal=True)), d["out_o"], "attn.o")
    ld, lds = H * Dh, H * S
    dv, dq, dk, dp = torch.empty_like(v), torch.empty_like(q), torch.empty_like(q), torch.empty_like(s16)
    gsb = ops.gemm_strided_batched
    gsb(True, False, H, S, Dh, S, 1.0, p16, lds, S, dO, ld, Dh, 0.0, dv, ld, Dh, 3)
    gsb(False, True, H, S, S, Dh, 1.0, dO, ld, Dh, v, ld, Dh, 0.0, dp, lds, S, 1)
    ds = ops.causal_softmax_bwd(s16, dp)
    gsb(True, False, H, S, Dh, S, alpha, ds, lds, S, q, ld, Dh, 0.0, dk, ld, Dh, 3)
    gsb(False, False, H, S, Dh, S, alpha, ds, lds, S, k, ld, Dh, 0.0, dq, ld, Dh, 2)
    close_enough(_host(dv), d["out_dv"], "attn.dv")
    close_enough(_host(dq), d["out_dq"], "attn.dq")
    close_enough(_host(dk), d["out_dk"], "attn.dk")


def _same_bits(got, want, name):
    got = np.ascontiguousarray(got)
    assert got.dtype.itemsize == want.dtype.itemsize and got.size == want.size, name
    assert got.tobytes() == np.ascontiguousarray(want).tobytes(), name


@pytest.mark.gpu
def test_gpu_digests_optimizer_and_raw_casts_hit_fixtures_bit_for_bit(ops):
    import torch
    d = load("digests")
    x = _dev(d["in_x"])
    assert int(ops.nan_count(x)) == int(d["out_nan"].ravel()[0])
    _same_bits(_host(ops.abs_log2_hist8(x)), d["out_hist"], "hist")
    hist, nan = ops.digests([x, x[:100]])
    _same_bits(_host(hist[0]), d["out_hist"], "batched hist")
    assert int(nan[0]) == int(d["out_nan"].ravel()[0])

    d = load("optimizer")
    hy = d["in_hyper"]
    sc = ops.adamw32_scalars(int(hy[0]), *[float(v) for v in hy[1:]])
    _same_bits(np.array(sc, np.float32), d["out_scalars"], "scalars")
    grad = _dev(d["in_grad"])
    f = lambda k: torch.from_numpy(d[k].copy()).cuda()
    _same_bits(_host(ops.online_average_scale_(grad, f("in_avg"), sc[0], sc[1])), d["out_thunk_avg"], "avg thunk")
    _same_bits(_host(ops.online_average_square_scale_(grad, f("in_avg2"), sc[0], sc[2])), d["out_thunk_avg2"], "avg2 thunk")
    _same_bits(_host(ops.online_adamw_update_(f("in_avg"), f("in_avg2"), f("in_master"), sc[3], sc[4], sc[5], sc[6])),
               d["out_thunk_update"], "update thunk")
    _same_bits(_host(ops.cast_f32_f16(f("in_master") * 3000.0)), d["out_thunk_cast"], "cast thunk")
    avg, avg2, master = f("in_avg"), f("in_avg2"), f("in_master")
    param = torch.empty_like(grad)
    ops.adamw32_step_([grad], [avg], [avg2], [master], [param], sc)
    for got, key in ((avg, "out_avg"), (avg2, "out_avg2"), (master, "out_master"), (param, "out_param")):
        _same_bits(_host(got), d[key], key)

    d = load("raw_casts")
    bf = torch.from_numpy(d["in_bf16"].view(np.int16).copy()).cuda()
    _same_bits(_host(ops.raw_cast_bf16_f16(bf)), d["out_bf16_f16"], "bf16_f16")
    _same_bits(_host(ops.raw_cast_bf16_f32(bf)), d["out_bf16_f32"], "bf16_f32")
    _same_bits(_host(ops.raw_cast_f32_bf16(torch.from_numpy(d["in_f32"].copy()).cuda())), d["out_f32_bf16"], "f32_bf16")
    _same_bits(_host(ops.raw_cast_f16_bf16(_dev(d["in_f16"]))), d["out_f16_bf16"], "f16_bf16")


@pytest.mark.gpu
def test_gpu_cached_pass_hits_fixture():
    from cacti_amd.runtime import Ctx, Llama, LlamaCached
    spec = importlib.util.spec_from_file_location("make_fixtures", os.path.join(GOLDEN, "make_fixtures.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    c = mod.TINY
    d = load("llama_cached_tiny")
    ctx = Ctx(0, 1 << 28, True)
    m = Llama(ctx, c["S"], c["D"], c["H"], c["Dh"], c["F"], c["V"], c["L"], c["eps"])
    m.put_params_flat(d["in_param"])
    k = LlamaCached(m, c["S"])
    cuts = [int(v) for v in d["in_cuts"]]
    for a, b in zip(cuts[:-1], cuts[1:]):
        k.set_tokens(d["in_tok"])
        k.apply(a, b)
        got = k.outputs()
        assert_parity(got["logit"], d["out_logit"][a:b], "cached logit %d:%d" % (a, b))
        want = d["out_logit"][a:b].astype(np.float32)
        top2 = np.sort(want, axis=1)[:, -2:]
        clear = (top2[:, 1] - top2[:, 0]) > 0.02
        assert np.array_equal(got["tok"][clear], d["out_tok"][a:b][clear])
    k.close(); m.close(); ctx.close()


@pytest.mark.gpu
def test_gpu_tiny_step_hits_fixture(oracle):
    """The whole cycle (stage, vadd_vjp, compile, resume) on the spine against the frozen
    gradients.  oracle is used for the parameter layout only."""
    from cacti_amd.runtime import Ctx, Llama
    spec = importlib.util.spec_from_file_location("make_fixtures", os.path.join(GOLDEN, "make_fixtures.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    c = mod.TINY
    d = load("llama_tiny")
    ctx = Ctx(0, 1 << 28, True)
    m = Llama(ctx, c["S"], c["D"], c["H"], c["Dh"], c["F"], c["V"], c["L"], c["eps"])
    m.put_params_flat(d["in_param"])
    out = m.step_explicit(d["in_tok"], d["in_lm_tok"], d["in_scale"], want_prob=False)
    assert_parity(out["loss"], d["out_loss"], "loss", l2=1e-4, mx=1e-3)
    assert_parity(out["logit"], d["out_logit"], "logit")
    cfg = oracle.Cfg(c["S"], c["D"], c["H"], c["Dh"], c["F"], c["V"], c["L"], c["eps"])
    want = oracle.split_params(cfg, d["out_grad"])
    for name, g in m.grads().items():
        assert_parity(g, want[name], "grad " + name, l2=2e-3, mx=4e-2)   # 2 layers: summation-order floor
    m.close(); ctx.close()
