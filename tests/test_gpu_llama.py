"""End-to-end: the tiny LLaMA cycle staged on the spine (reset / stage / vadd_vjp / compile /
resume / resume_put) against the CPU oracle, every parameter gradient (MI355X)."""
import numpy as np
import pytest

from tests.llama_ref import make_inputs
from tests.util import assert_parity, rel_l2, max_rel

pytestmark = pytest.mark.gpu

TINY = dict(S=128, D=256, H=4, Dh=64, F=688, V=1024, L=2, eps=1e-6)


def _model(cfg, pool_bytes=1 << 30, pagelocked=True):
    from cacti_amd.runtime import Ctx, Llama
    ctx = Ctx(0, pool_bytes, pagelocked)
    m = Llama(ctx, cfg.S, cfg.D, cfg.H, cfg.Dh, cfg.F, cfg.V, cfg.L, cfg.eps)
    return ctx, m


def _compare(oracle, cfg, m, ref, env, tag):
    """Every gradient tensor of the device against the oracle's default run, held to the summation-order
    envelope (tests/envelope.py): no further from the oracle than the oracle's own runs with other valid
    fp32 summation orders are from each other, ratio <= 1.0 per tensor."""
    from tests.envelope import assert_inside_envelope
    grads = m.grads()
    assert len(grads) == 3 + 9 * cfg.L
    return assert_inside_envelope(grads, oracle.split_params(cfg, ref["grad"]), env, tag)


@pytest.mark.parametrize("attention", ["fused", "thunks"])
def test_tiny_llama_step_all_gradients(oracle, attention):
    """Healthy-range variant: norm weights ~N(1, 0.02), grad_scale 1024 (the example's); the attention
    block staged as the fused thunk and as the reference's chain of separate thunks."""
    cfg, flat, tok, lm_tok, scale = make_inputs(TINY, seed=0, norm_mean=1.0, grad_scale=1024.0)
    ref = oracle.llama_step(cfg, flat, tok, lm_tok, scale)
    ctx, m = _model(cfg)
    m.set_attention(attention)
    m.put_params_flat(flat)
    out = m.step_explicit(tok, lm_tok, scale, want_prob=True)
    assert_parity(out["loss"], ref["loss"], "loss", l2=1e-4, mx=1e-3)
    assert_parity(out["logit"], ref["logit"], "logit")
    assert np.mean(out["amax"] == ref["amax"]) > 0.99       # ties in f16 logits may differ
    assert abs(out["prob"].sum(1) - 1).max() < 1e-4
    from tests.envelope import order_envelope
    _, env = order_envelope(oracle, cfg, flat, tok, lm_tok, scale)
    _compare(oracle, cfg, m, ref, env, "healthy")
    # and against exact arithmetic (fp64 autograd): no further from the truth than the oracle is
    from tests.llama_ref import torch_step
    _, g64, _ = torch_step(cfg, oracle.split_params(cfg, flat), tok, lm_tok, scale)
    want = oracle.split_params(cfg, ref["grad"])
    for name, g in m.grads().items():
        assert rel_l2(g, g64[name]) <= 1.15 * rel_l2(want[name], g64[name]) + 1e-4, name
    names = ctx.log_names()
    assert names.count("yield_set") == 3 and "unlive" in names and "rms_norm_bwd" in names
    assert ("attention_bwd" in names) == (attention == "fused")
    assert ("causal_softmax_bwd" in names) == (attention == "thunks")
    # a second cycle on the same context (reset GCs the first one's cells) gives the same result
    g1 = m.grads()
    loss2 = m.step(tok, lm_tok, scale)
    assert np.array_equal(loss2, out["loss"])
    for name, g in m.grads().items():
        assert np.array_equal(g.view(np.uint16), g1[name].view(np.uint16)), name
    m.close(); ctx.close()


def test_grouped_products_are_the_separate_thunks_bit_for_bit():
    """Small shapes (every product through the register path): the grouped stagings of the projections and
    of their weight gradients (modes 1 and 2) give the loss and all gradients of the separate matmul thunks
    (mode 0), bit for bit."""
    cfg, flat, tok, lm_tok, scale = make_inputs(TINY, seed=3, norm_mean=1.0, grad_scale=1024.0)
    got = {}
    for groups in (0, 1, 2):
        ctx, m = _model(cfg)
        m.set_product_groups(groups)
        m.put_params_flat(flat)
        got[groups] = (m.step(tok, lm_tok, scale), m.grads())
        m.close(); ctx.close()
    for groups in (1, 2):
        assert np.array_equal(got[groups][0], got[0][0])
        for n, g in got[groups][1].items():
            assert np.array_equal(g.view(np.uint16), got[0][1][n].view(np.uint16)), (groups, n)


def test_tiny_llama_literal_config(oracle):
    """The reference's small training configuration as written: every weight ~N(0, 0.02), loss scale 1/(S-1).
    The q/k/gate/up/down gradients (1e-8 .. 1e-11) underflow f16 in the reference's own
    arithmetic, so those tensors are compared in absolute terms (f16 subnormal quanta)."""
    cfg, flat, tok, lm_tok, scale = make_inputs(TINY, seed=0)
    ref = oracle.llama_step(cfg, flat, tok, lm_tok, scale)
    ctx, m = _model(cfg)
    m.put_params_flat(flat)
    loss = m.step(tok, lm_tok, scale)
    assert_parity(loss, ref["loss"], "loss", l2=1e-4, mx=1e-3)
    want = oracle.split_params(cfg, ref["grad"])
    for name, g in m.grads().items():
        w = want[name].astype(np.float64)
        rms = np.sqrt(np.mean(w * w))
        if rms > 2.0 ** -14:                                  # normal f16 range
            assert_parity(g, want[name], name)
        else:
            # within a few f16 subnormal quanta (2^-24) everywhere
            assert np.max(np.abs(g.astype(np.float64) - w)) <= 8 * 2.0 ** -24, name
    m.close(); ctx.close()


def test_bad_token_is_an_error(oracle):
    from cacti_amd.ffi import CactiError
    cfg, flat, tok, lm_tok, scale = make_inputs(dict(TINY, S=16, L=1), seed=1)
    ctx, m = _model(cfg)
    m.put_params_flat(flat)
    bad = lm_tok.copy(); bad[3] = cfg.V
    with pytest.raises(CactiError) as e:
        m.step(tok, bad, scale)
    assert e.value.code == -3
    m.step(tok, lm_tok, scale)                                # the context stays usable
    m.close(); ctx.close()


@pytest.mark.parametrize("pagelocked", [True, False])
def test_capped_pool_spills_and_matches(oracle, pagelocked):
    """Pool capped below the step's footprint: live cells spill to host memory and are
    re-uploaded; results are bit-identical to the uncapped run."""
    cfg, flat, tok, lm_tok, scale = make_inputs(TINY, seed=2, norm_mean=1.0, grad_scale=1024.0)
    ctx, m = _model(cfg)
    m.put_params_flat(flat)
    loss_a = m.step(tok, lm_tok, scale)
    ga = m.grads()
    peak = ctx.stats()["pool_peak"]
    m.close(); ctx.close()
    cap = int(peak * 0.45)
    ctx, m = _model(cfg, pool_bytes=cap, pagelocked=pagelocked)
    m.put_params_flat(flat)
    loss_b = m.step(tok, lm_tok, scale)
    st = ctx.stats()
    print("peak %d cap %d evictions %d d2h %d h2d %d" % (peak, st["pool_cap"], st["n_evict"],
                                                       st["bytes_d2h"], st["bytes_h2d"]), flush=True)
    assert st["n_evict"] > 0 and st["bytes_d2h"] > 0 and st["pool_peak"] <= st["pool_cap"]
    assert np.array_equal(loss_a, loss_b)
    for name, g in m.grads().items():
        assert np.array_equal(g.view(np.uint16), ga[name].view(np.uint16)), name
    m.close(); ctx.close()


@pytest.mark.parametrize("capped", [False, True])
def test_digests_of_parameters_and_gradients(oracle, capped):
    """abs_log2_hist8 and nan_count of every parameter and gradient after a cycle, as the
    reference's example takes them (examples/open_llama_3b_train.rs:409-424): bit-exact against
    the oracle's digests of the same tensors; also with cells spilled to the host in between."""
    cfg, flat, tok, lm_tok, scale = make_inputs(TINY, seed=4, norm_mean=1.0, grad_scale=1024.0)
    ctx, m = _model(cfg)
    m.put_params_flat(flat)
    m.step(tok, lm_tok, scale)
    if capped:
        peak = ctx.stats()["pool_peak"]
        m.close(); ctx.close()
        ctx, m = _model(cfg, pool_bytes=int(peak * 0.45))
        m.put_params_flat(flat)
        m.step(tok, lm_tok, scale)
    grads = m.grads()
    gh, gn = m.digests(of_grads=True)
    ph, pn = m.digests(of_grads=False)
    want_p = oracle.split_params(cfg, flat)
    for i, (name, shape) in enumerate(m.params):
        assert np.array_equal(gh[i], oracle.abs_log2_hist8(grads[name])), name
        assert gn[i] == oracle.nan_count(grads[name]) == 0, name
        assert np.array_equal(ph[i], oracle.abs_log2_hist8(want_p[name])), name
        assert pn[i] == 0 and ph[i].sum() == int(np.prod(shape)), name
    m.close(); ctx.close()


@pytest.mark.parametrize("capped", [False, True])
def test_adamw_steps_between_cycles(oracle, capped):
    """The example's minibatch loop (examples/open_llama_3b_train.rs:230-268): master = cast(param),
    zeroed averages, then cycle -> AdamW32 step -> cycle -> step.  Averages, master weights and the
    f16 parameters are bit-exact against the oracle's thunks applied to the gradients the device
    produced; the embedding stays as it was when skipped; the second cycle runs on the updated
    parameters (its loss differs).  Also with a pool so small that the optimiser state spills."""
    opt = dict(grad_scale=1024.0, lr=2.0e-3, wd=0.1, a1=0.1, a2=0.05, eps=1.0e-5)
    cfg, flat, tok, lm_tok, scale = make_inputs(TINY, seed=6, norm_mean=1.0, grad_scale=1024.0)
    ctx, m = _model(cfg)
    m.put_params_flat(flat)
    m.step(tok, lm_tok, scale)
    if capped:
        peak = ctx.stats()["pool_peak"]
        m.close(); ctx.close()
        ctx, m = _model(cfg, pool_bytes=int(peak))          # the cycle fits, the f32 optimiser state does not
        m.put_params_flat(flat)
    want_p = oracle.split_params(cfg, flat)
    names = [n for n, _ in m.params]
    master = {n: want_p[n].astype(np.float32) for n in names}
    avg = {n: np.zeros(want_p[n].shape, np.float32) for n in names}
    avg2 = {n: np.zeros(want_p[n].shape, np.float32) for n in names}
    m.adamw_init()
    losses = []
    for it in (1, 2):
        losses.append(m.step(tok, lm_tok, scale))
        grads = m.grads()
        m.adamw_step(it, skip_embed=(it == 1), **opt)
        sc = oracle.adamw32_scalars(it, **opt)
        for i, n in enumerate(names):
            if it == 1 and n == "embed":
                p16 = want_p[n]
            else:
                avg[n], avg2[n], master[n], p16 = oracle.adamw32_step(grads[n], avg[n], avg2[n], master[n], sc)
                want_p[n] = p16
            assert np.array_equal(m.adamw_state(i, "grad_avg").view(np.uint32), avg[n].view(np.uint32)), (it, n)
            assert np.array_equal(m.adamw_state(i, "grad2_avg").view(np.uint32), avg2[n].view(np.uint32)), (it, n)
            assert np.array_equal(m.adamw_state(i, "master").view(np.uint32), master[n].view(np.uint32)), (it, n)
            assert np.array_equal(m.param(i).view(np.uint16), p16.view(np.uint16)), (it, n)
    assert not np.array_equal(losses[0], losses[1])
    if capped:
        assert ctx.stats()["n_evict"] > 0
    from cacti_amd.ffi import CactiError
    with pytest.raises(CactiError) as e:
        m.adamw_step(0, **opt)
    assert e.value.code == -1
    m.close(); ctx.close()


def test_training_cycles_follow_the_oracle(oracle):
    """The example's loop end to end (examples/open_llama_3b_train.rs:223-531 with one cycle per
    minibatch): cycle -> AdamW32 step on every parameter but the embedding -> cycle ...; four cycles on
    the device against four cycles of the oracle (its own gradients, its own optimiser): per-cycle
    losses agree, the loss of the repeated batch goes down, and the parameters stay together."""
    opt = dict(grad_scale=1024.0, lr=1.0e-3, wd=0.1, a1=0.1, a2=0.05, eps=1.0e-5)
    cfg, flat, tok, lm_tok, scale = make_inputs(TINY, seed=9, norm_mean=1.0, grad_scale=1024.0)
    ctx, m = _model(cfg)
    m.put_params_flat(flat)
    m.adamw_init()
    names = [n for n, _ in m.params]
    o_p = {n: v.copy() for n, v in oracle.split_params(cfg, flat).items()}
    o_master = {n: o_p[n].astype(np.float32) for n in names}
    o_avg = {n: np.zeros(o_p[n].shape, np.float32) for n in names}
    o_avg2 = {n: np.zeros(o_p[n].shape, np.float32) for n in names}
    live = scale > 0
    g_losses, o_losses = [], []
    for it in range(1, 5):
        g_loss = m.step(tok, lm_tok, scale)
        m.adamw_step(it, skip_embed=True, **opt)
        oflat = np.concatenate([o_p[n].reshape(-1) for n in names])
        ref = oracle.llama_step(cfg, oflat, tok, lm_tok, scale)
        og = oracle.split_params(cfg, ref["grad"])
        sc = oracle.adamw32_scalars(it, **opt)
        for n in names[1:]:
            o_avg[n], o_avg2[n], o_master[n], o_p[n] = oracle.adamw32_step(og[n], o_avg[n], o_avg2[n], o_master[n], sc)
        g_losses.append(float(g_loss[live].mean()))
        o_losses.append(float(ref["loss"][live].mean()))
        assert abs(g_losses[-1] - o_losses[-1]) < 2e-3 * abs(o_losses[-1]), (it, g_losses, o_losses)
    assert g_losses[-1] < g_losses[0] - 0.05 and o_losses[-1] < o_losses[0] - 0.05, (g_losses, o_losses)
    for i, n in enumerate(names):
        got, want = m.param(i), o_p[n]
        if n == "embed":
            assert np.array_equal(got.view(np.uint16), want.view(np.uint16))
            continue
        # the step of one cycle is ~lr per element: two runs whose gradients differ in the last
        # bits stay within a small fraction of the total movement
        moved = np.abs(want.astype(np.float32) - oracle.split_params(cfg, flat)[n].astype(np.float32)).max()
        diff = np.abs(got.astype(np.float32) - want.astype(np.float32)).max()
        assert moved > 1e-3 and diff <= 0.35 * moved, (n, moved, diff)
    m.close(); ctx.close()


def test_adamw_step_before_init_is_a_state_error(oracle):
    from cacti_amd.ffi import CactiError
    cfg, flat, tok, lm_tok, scale = make_inputs(TINY, seed=6)
    ctx, m = _model(cfg)
    with pytest.raises(CactiError) as e:
        m.adamw_step(1)
    assert e.value.code == -5
    m.close(); ctx.close()


def test_pool_too_small_is_a_clean_error(oracle):
    from cacti_amd.ffi import CactiError
    cfg, flat, tok, lm_tok, scale = make_inputs(TINY, seed=3)
    ctx, m = _model(cfg, pool_bytes=1 << 19)                  # the head's weight alone fills it
    m.put_params_flat(flat)
    with pytest.raises(CactiError) as e:
        m.step(tok, lm_tok, scale)
    assert e.value.code == -4
    assert "pinned by the running thunk" in str(e.value) and "largest free" in str(e.value)
    # the usage table by class of cell (the reference dumps it before it panics, src/pctx/nvgpu.rs:2424-2440)
    rep = ctx.usage_report()
    print(rep)
    lines = rep.splitlines()
    assert lines[0].startswith("pool: cap=%d " % (1 << 19))
    assert [l.split()[0] for l in lines[1:6]] == ["parameters", "gradients", "optimiser", "tables,", "cycle"]
    n_par = int(lines[1].split("cells=")[1].split()[0])
    assert n_par == 3 + 9 * cfg.L and int(lines[2].split("cells=")[1].split()[0]) == n_par
    m.close(); ctx.close()


def test_full_size_step_properties():
    """The reference's 3B configuration at full shapes (S=2048, D=3200, H=32 x 100, F=8640, V=32000) with
    4 of the 26 layers (the oracle would need a minute per layer): properties that hold at any
    size.  (a) the loss is -log softmax(logit)[target] of the logits the step returns, recomputed
    in fp64; (b) a second cycle is bit-identical; (c) doubling the loss scale (a power of two)
    doubles the gradients: every product and sum on the adjoint path is homogeneous in the
    scale, so elements differ only where a value on the way was an f16 subnormal; (d) embedding rows
    of ids that do not occur get a zero gradient, rows that occur a non-zero one."""
    import bench
    from cacti_amd.runtime import Ctx, Llama
    cfg = dict(bench.LLAMA_3B, L=4)
    ctx = Ctx(0, 24 << 30, True)
    m = Llama(ctx, **cfg)
    bench.synth_params(m)
    tok, lm_tok, scale = bench.synth_inputs(cfg, grad_scale=8192.0)
    out = m.step_explicit(tok, lm_tok, scale)
    lg = out["logit"].astype(np.float64)
    lse = np.log(np.exp(lg - lg.max(1, keepdims=True)).sum(1)) + lg.max(1)
    want_loss = lse - lg[np.arange(cfg["S"]), lm_tok]
    assert np.all(np.isfinite(out["loss"]))
    assert np.abs(out["loss"] - want_loss).max() < 2e-3 * max(1.0, np.abs(want_loss).max())
    assert np.mean(out["amax"] == lg.argmax(1)) > 0.999

    idx = {name: i for i, (name, _) in enumerate(m.params)}
    probe = ["embed", "l0.q", "l0.pre_norm", "l1.down", "l3.gate", "l3.v", "head_norm", "lm_head"]
    g1 = {n: m.grad(idx[n]) for n in probe}
    m.step(tok, lm_tok, scale, want_loss=False)
    for n in probe:
        assert np.array_equal(m.grad(idx[n]).view(np.uint16), g1[n].view(np.uint16)), n

    present = np.zeros(cfg["V"], bool)
    present[tok] = True
    rows = np.abs(g1["embed"].astype(np.float32)).max(1)
    assert np.all(rows[~present] == 0) and np.mean(rows[present] > 0) > 0.99

    m.step(tok, lm_tok, 2.0 * scale, want_loss=False)
    tiny = 2.0 ** -14
    for n in probe:
        a, b = g1[n].astype(np.float32), m.grad(idx[n]).astype(np.float32)
        ok = (np.abs(a) >= tiny) & (np.abs(b) < 65504)
        assert ok.mean() > 0.03, (n, ok.mean())      # embed: only rows of ids that occur
        same = float(np.mean(b[ok] == 2.0 * a[ok]))
        err = rel_l2(b, 2.0 * a)
        print("scale x2: %-12s %.4f of the normal elements doubled exactly, rel_l2 %.2e" % (n, same, err),
              flush=True)
        assert err < 5e-3, (n, same, err)
    m.close(); ctx.close()


@pytest.mark.gpu
def test_cached_gradients_accumulate_micro_batches(oracle):
    """Two micro-batches with the gradients cached in between (g.cache(),
    examples/open_llama_3b_train.rs:334-345) against the oracle doing the same; caching before any cycle
    has written the gradients is an error; a plain cycle afterwards overwrites again."""
    from cacti_amd.ffi import CactiError
    cfg, flat, tok, lm_tok, scale = make_inputs(TINY, seed=0, norm_mean=1.0, grad_scale=1024.0)
    _, _, tok2, lm_tok2, _ = make_inputs(TINY, seed=17, norm_mean=1.0, grad_scale=1024.0)
    ctx, m = _model(cfg)
    m.put_params_flat(flat)
    with pytest.raises(CactiError) as e:
        m.step(tok, lm_tok, scale, accumulate=True)
    assert e.value.code == -5
    m.step(tok, lm_tok, scale)
    first = m.grads()
    loss2 = m.step(tok2, lm_tok2, scale, accumulate=True)
    a = oracle.llama_step(cfg, flat, tok, lm_tok, scale)
    ab = oracle.llama_step(cfg, flat, tok2, lm_tok2, scale, grad_cached=a["grad"])
    assert_parity(loss2, ab["loss"], "loss", l2=1e-4, mx=1e-3)
    from tests.envelope import assert_inside_envelope, order_envelope
    want = oracle.split_params(cfg, ab["grad"])
    got = m.grads()
    # the same rule as for one cycle: inside the envelope of the oracle's own summation orders, here of the
    # second cycle accumulating onto the oracle's first-cycle gradients
    _, env2 = order_envelope(oracle, cfg, flat, tok2, lm_tok2, scale, grad_cached=a["grad"])
    _, env1 = order_envelope(oracle, cfg, flat, tok, lm_tok, scale)
    env = {t: (env1[t][0] + env2[t][0], env1[t][1] + env2[t][1]) for t in env2}   # two free-running cycles
    assert_inside_envelope(got, want, env, "accumulated")
    for name, g in got.items():
        assert not np.array_equal(g, first[name]), name
    # from the device's own first gradients the accumulation adds exactly one micro-batch: got - first ~ b
    b = oracle.split_params(cfg, oracle.llama_step(cfg, flat, tok2, lm_tok2, scale)["grad"])
    for name, g in got.items():
        d = g.astype(np.float32) - first[name].astype(np.float32)
        assert rel_l2(d, b[name]) < 5e-3, name
    m.step(tok2, lm_tok2, scale)
    _, envb = order_envelope(oracle, cfg, flat, tok2, lm_tok2, scale)
    assert_inside_envelope(m.grads(), b, envb, "overwritten")
    m.close(); ctx.close()


@pytest.mark.gpu
def test_copy_forwarding_changes_no_bit(tmp_path):
    """The compile pass that turns the adjoint copies of a residual add into storage moves must not change
    any result: one cycle in a child process with the pass, one with CACTI_NO_COPY_FORWARD=1 (the switch is
    read once per process), gradients and loss compared byte for byte."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    code = (
        "import sys, numpy as np\n"
        "sys.path.insert(0, %r)\n"
        "from tests.llama_ref import make_inputs\n"
        "from tests.test_gpu_llama import TINY, _model\n"
        "cfg, flat, tok, lm_tok, scale = make_inputs(TINY, seed=4, norm_mean=1.0, grad_scale=1024.0)\n"
        "ctx, m = _model(cfg)\n"
        "m.put_params_flat(flat)\n"
        "loss = m.step(tok, lm_tok, scale)\n"
        "g = m.grads()\n"
        "np.savez(sys.argv[1], loss=loss, **{k: v.view(np.uint16) for k, v in g.items()})\n"
        "print(ctx.stats())\n" % root)
    outs = []
    for tag, extra in (("fwd", {}), ("plain", {"CACTI_NO_COPY_FORWARD": "1"})):
        path = str(tmp_path / (tag + ".npz"))
        env = dict(os.environ, **extra)
        r = subprocess.run([sys.executable, "-c", code, path], env=env, capture_output=True, text=True, timeout=110)
        assert r.returncode == 0, r.stderr[-2000:]
        outs.append(np.load(path))
    a, b = outs
    assert sorted(a.files) == sorted(b.files) and len(a.files) == 3 + 9 * TINY["L"] + 1
    for k in a.files:
        assert a[k].tobytes() == b[k].tobytes(), k


@pytest.mark.gpu
def test_capped_pool_spills_at_full_shapes():
    """The host-spill path at the OpenLLaMA-3B shapes (4 of the 26 layers): with the pool capped at 0.45 of
    the uncapped peak -- below what parameters and gradients alone take -- live cells are downloaded on the
    copy stream, victims chosen by their next use in the compiled log, and uploaded again ahead of their
    use; loss and every probed gradient are bit-identical to the uncapped run, over two cycles."""
    import bench
    from cacti_amd.runtime import Ctx, Llama
    cfg = dict(bench.LLAMA_3B, L=4)
    tok, lm_tok, scale = bench.synth_inputs(cfg, grad_scale=8192.0)
    probe = ["embed", "l0.q", "l0.pre_norm", "l1.down", "l2.up", "l3.gate", "l3.v", "head_norm", "lm_head"]

    def run(pool_bytes):
        ctx = Ctx(0, pool_bytes, True)
        m = Llama(ctx, **cfg)
        bench.synth_params(m)
        idx = {name: i for i, (name, _) in enumerate(m.params)}
        out = []
        for _ in range(2):
            loss = m.step(tok, lm_tok, scale)
            out.append((loss, {n: m.grad(idx[n]) for n in probe}))
        st = ctx.stats()
        m.close(); ctx.close()
        return out, st

    ref, st0 = run(24 << 30)
    assert st0["n_evict"] == 0
    cap = int(st0["pool_peak"] * 0.45)
    got, st = run(cap)
    print("peak %.2f GB, cap %.2f GB: %d evictions, %.2f GB down, %.2f GB up over two cycles"
          % (st0["pool_peak"] / 1e9, cap / 1e9, st["n_evict"], st["bytes_d2h"] / 1e9, st["bytes_h2d"] / 1e9), flush=True)
    assert st["n_evict"] > 0 and st["bytes_d2h"] > 0 and st["pool_peak"] <= st["pool_cap"]
    for cyc in range(2):
        assert np.array_equal(ref[cyc][0], got[cyc][0]), "loss, cycle %d" % cyc
        for n in probe:
            assert np.array_equal(ref[cyc][1][n].view(np.uint16), got[cyc][1][n].view(np.uint16)), (cyc, n)


def test_full_depth_step_on_a_16_gib_pool():
    """The whole 26-layer OpenLLaMA-3B-shaped step on a pool capped at 16 GiB (the reference's card,
    examples/open_llama_3b_train.rs): two cycles; the loss and twelve probed gradients (first and last
    layers, every kind of tensor, embedding and LM head) are bit-identical to the uncapped run's, and the
    capped run really spilled."""
    import bench
    from cacti_amd.runtime import Ctx, Llama
    cfg = dict(bench.LLAMA_3B)
    assert cfg["L"] == 26
    tok, lm_tok, scale = bench.synth_inputs(cfg)

    def run(pool_bytes):
        print("26 layers on a pool of %.0f GiB" % (pool_bytes / 2 ** 30), flush=True)
        ctx = Ctx(0, pool_bytes, True)
        m = Llama(ctx, **cfg)
        bench.synth_params(m)
        out = []
        for _ in range(2):
            loss = m.step(tok, lm_tok, scale)
            out.append((loss, bench.probe_grads(m, cfg)))
        st = ctx.stats()
        m.close(); ctx.close()
        return out, st

    got, st = run(bench.CAPPED_POOL_BYTES)
    ref, st0 = run(40 << 30)
    print("uncapped peak %.2f GB; at 16 GiB: %d evictions, %.2f GB down, %.2f GB up over two cycles"
          % (st0["pool_peak"] / 1e9, st["n_evict"], st["bytes_d2h"] / 1e9, st["bytes_h2d"] / 1e9), flush=True)
    assert st0["n_evict"] == 0
    assert st["n_evict"] > 0 and st["bytes_d2h"] > 0 and st["bytes_h2d"] > 0 and st["pool_peak"] <= st["pool_cap"]
    for cyc in range(2):
        assert np.all(np.isfinite(ref[cyc][0]))
        assert np.array_equal(ref[cyc][0], got[cyc][0]), "loss, cycle %d" % cyc
        assert len(ref[cyc][1]) >= 12
        for n, g in ref[cyc][1].items():
            assert np.array_equal(g.view(np.uint16), got[cyc][1][n].view(np.uint16)), (cyc, n)
