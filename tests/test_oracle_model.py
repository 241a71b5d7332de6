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
