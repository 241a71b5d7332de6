"""Composed model: the oracle's gradients for the tiny configuration against an
independent fp64 torch.autograd statement of the same model (no GPU needed)."""
import numpy as np

from tests.llama_ref import make_inputs, torch_step
from tests.util import rel_l2, max_rel

TINY = dict(S=128, D=256, H=4, Dh=64, F=688, V=1024, L=2, eps=1e-6)


def test_tiny_llama_gradients_vs_fp64_autograd(oracle):
    # norm weights ~N(1, 0.02) and the example's grad_scale 1024 keep every gradient in the
    # normal f16 range; with all weights ~N(0, 0.02) the q/k gradients (~1e-10) underflow f16
    cfg, flat, tok, lm_tok, scale = make_inputs(TINY, seed=0, norm_mean=1.0, grad_scale=1024.0)
    out = oracle.llama_step(cfg, flat, tok, lm_tok, scale)
    params = oracle.split_params(cfg, flat)
    grads = oracle.split_params(cfg, out["grad"])
    loss64, g64, logit64 = torch_step(cfg, params, tok, lm_tok, scale)
    assert rel_l2(out["loss"], loss64) < 1e-3
    assert rel_l2(out["logit"], logit64) < 3e-3
    worst = 0.0
    for name, g in grads.items():
        assert g.shape == g64[name].shape
        e = rel_l2(g, g64[name])
        worst = max(worst, e)
        # a chain of individually rounded f16 thunks against exact arithmetic:
        # tolerance-level agreement, not bit-level
        assert e < 3e-3 and max_rel(g, g64[name]) < 5e-2, (name, e)
    assert len(grads) == 3 + 9 * cfg.L
    print("worst rel_l2 vs fp64 autograd: %.3e" % worst)


def test_out_of_range_token_is_an_error(oracle):
    cfg, flat, tok, lm_tok, scale = make_inputs(dict(TINY, S=16, L=1), seed=1)
    import pytest
    bad = lm_tok.copy(); bad[3] = cfg.V
    with pytest.raises(IndexError):
        oracle.llama_step(cfg, flat, tok, bad, scale)


def test_summation_order_floor_of_the_f16_chain(oracle):
    """Two equally valid restatements (GEMMs summed in ascending / descending k) differ by
    ~1e-3 relative L2 after two layers: fp32 order changes become independent f16 rounding
    flips that every later GEMM re-amplifies.  No implementation with another summation
    order (cuBLAS, MFMA) can agree with the oracle more closely than this."""
    cfg, flat, tok, lm_tok, scale = make_inputs(TINY, seed=0, norm_mean=1.0, grad_scale=1024.0)
    a = oracle.llama_step(cfg, flat, tok, lm_tok, scale)
    oracle.set_gemm_reverse_k(1)
    try:
        b = oracle.llama_step(cfg, flat, tok, lm_tok, scale)
    finally:
        oracle.set_gemm_reverse_k(0)
    ga, gb = oracle.split_params(cfg, a["grad"]), oracle.split_params(cfg, b["grad"])
    floors = [rel_l2(gb[n], ga[n]) for n in ga]
    print("order floor: min %.2e max %.2e" % (min(floors), max(floors)))
    assert 2e-4 < min(floors) and max(floors) < 3e-3
    assert rel_l2(b["loss"], a["loss"]) < 1e-4


def test_cached_gradients_accumulate_micro_batches(oracle):
    """g.cache() before a cycle (examples/open_llama_3b_train.rs:334-345) makes the cycle's first write into
    every gradient an accumulation.  Pins: cached zeros change nothing, bit for bit (f16(x + 0) = x for the
    beta = 1 products and for the y = oy + y thunks alike); two micro-batches give, within f16 rounding of
    the sum, the fp64 autograd gradient of the two-batch loss."""
    cfg, flat, tok, lm_tok, scale = make_inputs(TINY, seed=0, norm_mean=1.0, grad_scale=1024.0)
    _, _, tok2, lm_tok2, _ = make_inputs(TINY, seed=17, norm_mean=1.0, grad_scale=1024.0)
    a = oracle.llama_step(cfg, flat, tok, lm_tok, scale)
    z = oracle.llama_step(cfg, flat, tok, lm_tok, scale, grad_cached=np.zeros_like(a["grad"]))
    assert np.array_equal(z["grad"].view(np.uint16), a["grad"].view(np.uint16))
    assert np.array_equal(z["loss"], a["loss"])
    ab = oracle.llama_step(cfg, flat, tok2, lm_tok2, scale, grad_cached=a["grad"])
    b = oracle.llama_step(cfg, flat, tok2, lm_tok2, scale)
    assert np.array_equal(ab["loss"], b["loss"])                       # the forward pass does not see the cache
    params = oracle.split_params(cfg, flat)
    _, ga64, _ = torch_step(cfg, params, tok, lm_tok, scale)
    _, gb64, _ = torch_step(cfg, params, tok2, lm_tok2, scale)
    got = oracle.split_params(cfg, ab["grad"])
    ga, gb = oracle.split_params(cfg, a["grad"]), oracle.split_params(cfg, b["grad"])
    for name, g in got.items():
        assert rel_l2(g, ga64[name] + gb64[name]) < 3e-3, name
        # against the sum of the two separately rounded gradients: one more f16 rounding at most
        want = ga[name].astype(np.float32) + gb[name].astype(np.float32)
        assert rel_l2(g, want) < 6e-4 and max_rel(g, want) < 2e-3, name


def test_python_trace_reproduces_the_c_composition(oracle):
    """tests/teacher.py composes the cycle from the oracle's per-thunk functions and records every
    call; its loss and 21 gradients must be those of oracle_llama_step bit for bit, which is what
    lets a device test replay the recorded calls one thunk at a time."""
    from tests.teacher import trace_step
    cfg, flat, tok, lm_tok, scale = make_inputs(TINY, seed=0, norm_mean=1.0, grad_scale=1024.0)
    ref = oracle.llama_step(cfg, flat, tok, lm_tok, scale)
    calls, loss, grads = trace_step(cfg, flat, tok, lm_tok, scale)
    assert np.array_equal(loss, ref["loss"])
    want = oracle.split_params(cfg, ref["grad"])
    assert sorted(grads) == sorted(want)
    for name, g in grads.items():
        assert np.array_equal(g.view(np.uint16), want[name].view(np.uint16)), name
    kinds = {c.kind for c in calls}
    assert kinds >= {"matmul", "block_matmul", "rms_norm_fwd", "rms_norm_bwd", "rope_fwd", "rope_bwd",
                     "silu_gate_fwd", "silu_gate_bwd", "causal_softmax_fwd", "causal_softmax_bwd",
                     "softmax_ce_fwd", "softmax_ce_bwd", "embed_fwd", "embed_bwd", "add"}
    # 7 forward + 14 backward products per layer, 1 + 2 for the head
    assert sum(c.kind == "matmul" for c in calls) == 21 * cfg.L + 3


def test_summation_order_envelope(oracle):
    """Twelve restatements of the cycle that differ only in what the reference leaves open (eight fp32
    summation orders of the GEMMs: ascending, descending, in blocks, pairwise; f32 instead of f64
    reductions; correctly rounded exp / log): every pair of them lands 0.6-1.3e-3 apart per gradient
    tensor after two layers, none of them is special.  The largest pairwise distance per tensor is the envelope the device
    result is held to.  A one-ulp change elsewhere (the norm's x / r as x * (1 / r)) moves the result
    just as far, which is why the device kernels keep the reference's operations where they can."""
    from tests.envelope import order_envelope
    cfg, flat, tok, lm_tok, scale = make_inputs(TINY, seed=0, norm_mean=1.0, grad_scale=1024.0)
    runs, env = order_envelope(oracle, cfg, flat, tok, lm_tok, scale)
    assert len(runs) == 12
    l2s = [e[0] for e in env.values()]
    print("envelope rel_l2: min %.2e max %.2e" % (min(l2s), max(l2s)))
    assert 4e-4 < min(l2s) and max(l2s) < 2e-3
    oracle.set_norm_reciprocal(1)
    try:
        alt = oracle.split_params(cfg, oracle.llama_step(cfg, flat, tok, lm_tok, scale)["grad"])
    finally:
        oracle.set_norm_reciprocal(0)
    moved = max(rel_l2(alt[n], runs["ascending"][n]) for n in alt)
    assert 5e-4 < moved < 3e-3
