"""Writes tests/golden/*.npz: small seeded inputs and the CPU oracle's outputs for every unit of
the path (fused adjoint kernels, the four GEMM layouts, the attention block, one tiny model step).

The reference holds no golden vectors for this path and cannot be run here, so these vectors
are the oracle's own output, frozen: what pins the oracle is the mathematics in
tests/test_oracle_thunks.py and tests/test_oracle_model.py.  The fixtures guard against the
oracle drifting (tests/test_golden.py, CPU) and give the HIP path fixed vectors to hit (GPU).

f16 tensors are stored as their uint16 bit patterns.  Run from the repository root:
    python tests/golden/make_fixtures.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import oracle  # noqa: E402
from tests.llama_ref import make_inputs  # noqa: E402

TINY = dict(S=16, D=32, H=2, Dh=16, F=40, V=64, L=2, eps=1e-6)


def randn16(r, shape, std=1.0):
    return (r.standard_normal(shape) * std).astype(np.float16)


def bits(a):
    a = np.ascontiguousarray(a)
    return a.view(np.uint16) if a.dtype == np.float16 else a


def units():
    """name -> dict of arrays (inputs prefixed in_, oracle outputs out_)."""
    r = np.random.default_rng(20240607)
    out = {}

    x, w, dy = randn16(r, (6, 64)), randn16(r, (64,), 0.1) + np.float16(1), randn16(r, (6, 64))
    y, _, _ = oracle.rmsnorm_fwd(x, w, 1e-6)
    dx, dw = oracle.rmsnorm_bwd(x, w, 1e-6, dy)
    dx0, dw0 = randn16(r, (6, 64)), randn16(r, (64,))
    dxa, dwa = oracle.rmsnorm_bwd(x, w, 1e-6, dy, dx0, dw0)
    out["rmsnorm"] = dict(in_x=x, in_w=w, in_dy=dy, in_dx0=dx0, in_dw0=dw0, out_y=y, out_dx=dx,
                          out_dw=dw, out_dx_acc=dxa, out_dw_acc=dwa)

    for tag, (S, H, Dh) in {"rope_dh12": (8, 2, 12), "rope_dh100": (4, 4, 100)}.items():
        cos, sin = oracle.rope_tables(S, Dh)
        x, dy, dx0 = randn16(r, (S, H, Dh)), randn16(r, (S, H, Dh)), randn16(r, (S, H, Dh))
        out[tag] = dict(in_x=x, in_dy=dy, in_dx0=dx0, out_cos=cos, out_sin=sin,
                        out_y=oracle.rope_fwd(x, cos, sin), out_dx=oracle.rope_bwd(dy, cos, sin),
                        out_dx_acc=oracle.rope_bwd(dy, cos, sin, dx0))

    g, u, dh = randn16(r, (512,), 2.0), randn16(r, (512,)), randn16(r, (512,))
    dg0, du0 = randn16(r, (512,)), randn16(r, (512,))
    _, hh = oracle.silu_gate_fwd(g, u)
    dg, du = oracle.silu_gate_bwd(g, u, dh)
    dga, dua = oracle.silu_gate_bwd(g, u, dh, dg0, du0)
    out["silu_gate"] = dict(in_g=g, in_u=u, in_dh=dh, in_dg0=dg0, in_du0=du0, out_h=hh, out_dg=dg,
                            out_du=du, out_dg_acc=dga, out_du_acc=dua)

    s16, dp = randn16(r, (16, 2, 16), 2.0), randn16(r, (16, 2, 16))
    out["causal_softmax"] = dict(in_s16=s16, in_dp16=dp, out_p16=oracle.causal_softmax_fwd(s16),
                                 out_ds16=oracle.causal_softmax_bwd(s16, dp))

    logit = randn16(r, (4, 40), 3.0)
    tok = r.integers(0, 40, 4).astype(np.uint16)
    scale = np.array([0.0, 0.5, 1.0, 2.0], np.float32)
    prob, loss, amax = oracle.softmax_ce_fwd(logit, tok)
    out["softmax_ce"] = dict(in_logit=logit, in_tok=tok, in_scale=scale, out_prob=prob, out_loss=loss,
                             out_amax=amax, out_dlogit=oracle.softmax_ce_bwd(logit, tok, scale))

    W = randn16(r, (16, 8))
    idx = np.array([3, 3, 0, 15, 7, 3, 0, 9, 9, 1, 2, 15], np.uint16)      # duplicates on purpose
    dy = randn16(r, (12, 8))
    out["embed"] = dict(in_W=W, in_idx=idx, in_dy=dy, out_y=oracle.embed_fwd(W, idx),
                        out_dW=oracle.embed_bwd(16, idx, dy))

    M, N, K = 24, 16, 20
    C0 = randn16(r, (M, N))
    d = dict(in_C0=C0)
    for ta in (0, 1):
        for tb in (0, 1):
            A = randn16(r, (K, M) if ta else (M, K))
            B = randn16(r, (N, K) if tb else (K, N))
            t = "NT"[ta] + "NT"[tb]
            d["in_A_" + t], d["in_B_" + t] = A, B
            d["out_C_" + t] = oracle.matmul(ta, tb, A, B)
            d["out_Cacc_" + t] = oracle.matmul(ta, tb, A, B, 0.25, 1.0, C0)
    out["matmul"] = d

    q, k, v, dO = (randn16(r, (16, 2, 12)) for _ in range(4))
    alpha = 1.0 / np.sqrt(12.0)
    s16, p16, o = oracle.attention_fwd(q, k, v, alpha)
    dq, dk, dv = oracle.attention_bwd(q, k, v, dO, alpha)
    out["attention"] = dict(in_q=q, in_k=k, in_v=v, in_dO=dO, in_alpha=np.float32(alpha),
                            out_s16=s16, out_p16=p16, out_o=o, out_dq=dq, out_dk=dk, out_dv=dv)

    cfg, flat, tok, lm_tok, scale = make_inputs(TINY, seed=3, norm_mean=1.0, grad_scale=1024.0)
    ref = oracle.llama_step(cfg, flat, tok, lm_tok, scale)
    out["llama_tiny"] = dict(in_param=flat, in_tok=tok, in_lm_tok=lm_tok, in_scale=scale,
                             out_loss=ref["loss"], out_logit=ref["logit"], out_amax=ref["amax"],
                             out_grad=ref["grad"])
    return out


def main():
    for name, d in units().items():
        path = os.path.join(HERE, name + ".npz")
        np.savez_compressed(path, **{k: bits(np.asarray(v)) for k, v in d.items()})
        print("%-16s %6d bytes" % (name, os.path.getsize(path)))


if __name__ == "__main__":
    main()
