"""Writes tests/golden/*.npz: small seeded inputs and the CPU oracle's outputs for every unit of
the path (fused adjoint kernels, the four GEMM layouts, the attention block, one tiny model step)
and of the rows around it (digests, optimiser thunks and one AdamW32 step, the bf16 raw casts, the
key / value-cached forward pass).

The reference holds no golden vectors for this path and cannot be run here, so these vectors
are the oracle's own output, frozen: what pins the oracle is the mathematics in
tests/test_oracle_thunks.py and tests/test_oracle_model.py.  The fixtures guard against the
oracle drifting (tests/test_golden.py, CPU) and give the HIP path fixed vectors to hit (GPU).

f16 tensors are stored as their uint16 bit patterns (bf16 patterns and token ids are genuine uint16:
tests/test_golden.py lists those names).  Run from the repository root:
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
    out.update(next_rows(r, cfg, flat, tok))
    return out


def next_rows(r, cfg, flat, tok):
    """digests, optimiser thunks, raw casts, cached forward pass"""
    out = {}
    # every exponent class, both signs, zeros, denormals, infinities, quiet and signalling NaNs
    pat = np.concatenate([r.integers(0, 65536, 3000), np.arange(0, 65536, 1024), [0, 0x8000, 1, 0x8001, 0x03ff, 0x0400,
                          0x7c00, 0xfc00, 0x7c01, 0x7e00, 0xfe00, 0x7fff, 0xffff, 0x7bff]]).astype(np.uint16)
    x = pat.view(np.float16)
    out["digests"] = dict(in_x=x, out_nan=np.int64(oracle.nan_count(x)), out_hist=oracle.abs_log2_hist8(x))

    n = 777
    grad = randn16(r, (n,), 300.0)
    grad[:3] = [0.0, 65504.0, -65504.0]
    avg, avg2 = (r.standard_normal(n) * 0.1).astype(np.float32), (r.random(n) * 0.1).astype(np.float32)
    avg2[3:6] = [0.0, 1e-30, 4.0]
    master = (r.standard_normal(n) * 0.02).astype(np.float32)
    hyper = dict(iter_nr=3, grad_scale=1024.0, lr=2e-5, wd=0.1, a1=0.1, a2=0.05, eps=1e-5)
    sc = oracle.adamw32_scalars(**hyper)
    navg, navg2, nmaster, nparam = oracle.adamw32_step(grad, avg, avg2, master, sc)
    out["optimizer"] = dict(
        in_grad=grad, in_avg=avg, in_avg2=avg2, in_master=master,
        in_hyper=np.array([hyper[k] for k in ("iter_nr", "grad_scale", "lr", "wd", "a1", "a2", "eps")], np.float64),
        out_scalars=sc, out_avg=navg, out_avg2=navg2, out_master=nmaster, out_param=nparam,
        out_thunk_avg=oracle.online_average_scale(grad, avg, sc[0], sc[1]),
        out_thunk_avg2=oracle.online_average_square_scale(grad, avg2, sc[0], sc[2]),
        out_thunk_update=oracle.online_adamw_update(avg, avg2, master, sc[3], sc[4], sc[5], sc[6]),
        out_thunk_cast=oracle.cast_f32_f16(master * 3000.0))

    bf = np.concatenate([r.integers(0, 65536, 2000), np.arange(0, 65536, 512)]).astype(np.uint16)
    f32 = np.concatenate([r.standard_normal(1000) * 10.0 ** r.integers(-42, 39, 1000),
                          [0.0, -0.0, np.inf, -np.inf, np.nan, 65504.0, 1e-45, 3.4e38]]).astype(np.float32)
    h16 = np.concatenate([r.integers(0, 65536, 2000), np.arange(0, 65536, 512)]).astype(np.uint16).view(np.float16)
    out["raw_casts"] = dict(in_bf16=bf, in_f32=f32, in_f16=h16,
                            out_bf16_f16=oracle.raw_cast("bf16_f16", bf), out_bf16_f32=oracle.raw_cast("bf16_f32", bf),
                            out_f32_bf16=oracle.raw_cast("f32_bf16", f32), out_f16_bf16=oracle.raw_cast("f16_bf16", h16))

    # the cached pass on the tiny model's parameters: a prompt of 5, one position, the other 10
    kc, vc = oracle.llama_cached_state(cfg)
    logits, toks = [], []
    cuts = [0, 5, 6, cfg.S]
    for a, b in zip(cuts[:-1], cuts[1:]):
        got = oracle.llama_cached_apply(cfg, flat, kc, vc, tok.copy(), a, b)
        logits.append(got["logit"])
        toks.append(got["tok"])
    out["llama_cached_tiny"] = dict(in_param=flat, in_tok=tok, in_cuts=np.array(cuts, np.int64),
                                    out_logit=np.concatenate(logits), out_tok=np.concatenate(toks),
                                    out_k_cache=kc, out_v_cache=vc)
    return out


def main():
    for name, d in units().items():
        path = os.path.join(HERE, name + ".npz")
        np.savez_compressed(path, **{k: bits(np.asarray(v)) for k, v in d.items()})
        print("%-16s %6d bytes" % (name, os.path.getsize(path)))


if __name__ == "__main__":
    main()
