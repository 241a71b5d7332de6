"""The LLaMA cycle re-composed in Python from the oracle's per-thunk functions, keeping every
thunk's inputs and outputs (test helper).

`oracle_llama_step` composes the same units in C (src/librarium/llama.rs:420-548 forward, the
adjoint pass of src/spine.rs:447-690 in reverse log order).  `trace_step` must reproduce its loss
and gradients bit for bit (a CPU test asserts that), which pins this composition; the recorded
calls are then what a *teacher-forced* device test replays: each HIP thunk gets the oracle's own
inputs, so its output is compared at the literal tolerance with no compounding of rounding flips
through the chain.
"""
import numpy as np

from oracle import oracle as o


class Call:
    """One thunk (or fused unit) application: kind, keyword inputs, named outputs."""

    def __init__(self, kind, where, ins, outs):
        self.kind, self.where, self.ins, self.outs = kind, where, ins, outs

    def __repr__(self):
        return "%s@%s" % (self.kind, self.where)


def _c(a):
    return np.ascontiguousarray(a)


def trace_step(cfg, flat, tok, lm_tok, scale, sink=None):
    """Returns (calls, loss, grads dict).  Every array in a Call is a private copy.  With `sink`, each Call is
    handed to sink(call) as soon as it is recorded instead of being kept (large shapes: the trace of one
    3B-shaped layer is several GB) and the returned list is empty."""
    S, D, H, Dh, F, V, L = cfg.S, cfg.D, cfg.H, cfg.Dh, cfg.F, cfg.V, cfg.L
    eps = float(cfg.eps)
    alpha = float(np.float32(1.0) / np.sqrt(np.float32(Dh)))
    P = o.split_params(cfg, flat)
    cos, sin = o.rope_tables(S, Dh)
    calls = []

    def rec(kind, where, ins, outs):
        c = Call(kind, where, {k: (v.copy() if isinstance(v, np.ndarray) else v) for k, v in ins.items()},
                 {k: v.copy() for k, v in outs.items()})
        if sink is None:
            calls.append(c)
        else:
            sink(c)

    def mm(where, ta, tb, A, B, alpha_=1.0, beta=0.0, C_init=None):
        out = o.matmul(ta, tb, A, B, alpha_, beta, C_init)
        rec("matmul", where, dict(ta=ta, tb=tb, A=A, B=B, alpha=alpha_, beta=beta, C_init=C_init), dict(C=out))
        return out

    def bmm(where, ta, tb, M, N, K, alpha_, A, lda, sa, B, ldb, sb, shape, ldc, sc, tri):
        out = np.zeros(shape, np.float16)
        o.block_matmul(ta, tb, H, M, N, K, alpha_, A, lda, sa, B, ldb, sb, 0.0, out, ldc, sc)
        rec("block_matmul", where, dict(ta=ta, tb=tb, M=M, N=N, K=K, alpha=alpha_, A=A, lda=lda, sa=sa, B=B,
                                        ldb=ldb, sb=sb, ldc=ldc, sc=sc, tri=tri), dict(C=out))
        return out

    def norm_f(where, x, w):
        y, _, _ = o.rmsnorm_fwd(x, w, eps)
        rec("rms_norm_fwd", where, dict(x=x, w=w, eps=eps), dict(y=y))
        return y

    def norm_b(where, x, w, dy, dx_init):
        dx, dw = o.rmsnorm_bwd(x, w, eps, dy, dx_init=dx_init)
        rec("rms_norm_bwd", where, dict(x=x, w=w, eps=eps, dy=dy, dx_init=dx_init), dict(dx=dx, dw=dw))
        return dx, dw

    def rope_f(where, x):
        y = o.rope_fwd(_c(x.reshape(S, H, Dh)), cos, sin).reshape(S, D)
        rec("rope_fwd", where, dict(x=x.reshape(S, H, Dh), cos=cos, sin=sin), dict(y=y.reshape(S, H, Dh)))
        return y

    def rope_b(where, dy):
        dx = o.rope_bwd(_c(dy.reshape(S, H, Dh)), cos, sin).reshape(S, D)
        rec("rope_bwd", where, dict(dy=dy.reshape(S, H, Dh), cos=cos, sin=sin), dict(dx=dx.reshape(S, H, Dh)))
        return dx

    def add(where, a, b):
        y = o.accumulate_f16(a, b)
        rec("add", where, dict(a=a, b=b), dict(y=y))
        return y

    ld, lds = H * Dh, H * S
    stream = o.embed_fwd(P["embed"], tok)
    rec("embed_fwd", "embed", dict(W=P["embed"], tok=tok), dict(y=stream))
    saved = []
    for l in range(L):
        g = lambda n: P["l%d.%s" % (l, n)]
        w = "l%d." % l
        x0 = stream
        pre = norm_f(w + "pre_norm", x0, g("pre_norm"))
        q = mm(w + "q", 0, 1, pre, g("q"))
        qr = rope_f(w + "q", q)
        k = mm(w + "k", 0, 1, pre, g("k"))
        kr = rope_f(w + "k", k)
        v = mm(w + "v", 0, 1, pre, g("v"))
        s16 = bmm(w + "qk", 0, 1, S, S, Dh, alpha, qr, ld, Dh, kr, ld, Dh, (S, H, S), lds, S, 1)
        p16 = o.causal_softmax_fwd(s16)
        rec("causal_softmax_fwd", w + "softmax", dict(s16=s16), dict(p16=p16))
        attn = bmm(w + "pv", 0, 0, S, Dh, S, 1.0, p16, lds, S, v, ld, Dh, (S, D), ld, Dh, 2)
        rec("attention_fwd", w + "attention", dict(q=qr.reshape(S, H, Dh), k=kr.reshape(S, H, Dh),
                                                   v=v.reshape(S, H, Dh), alpha=alpha), dict(o=attn.reshape(S, H, Dh)))
        oo = mm(w + "o", 0, 1, attn, g("o"))
        x1 = add(w + "x1", x0, oo)
        post = norm_f(w + "post_norm", x1, g("post_norm"))
        up = mm(w + "up", 0, 1, post, g("up"))
        gate = mm(w + "gate", 0, 1, post, g("gate"))
        _, h = o.silu_gate_fwd(gate, up)
        rec("silu_gate_fwd", w + "silu_gate", dict(g=gate, u=up), dict(h=h))
        down = mm(w + "down", 0, 1, h, g("down"))
        stream = add(w + "x2", x1, down)
        saved.append(dict(x0=x0, pre=pre, qr=qr, kr=kr, v=v, s16=s16, p16=p16, attn=attn, x1=x1, post=post, up=up,
                          gate=gate, h=h))
    hn = norm_f("head_norm", stream, P["head_norm"])
    logit = mm("lm_head", 0, 1, hn, P["lm_head"])
    _, loss, amax = o.softmax_ce_fwd(logit, lm_tok, want_prob=False)
    rec("softmax_ce_fwd", "loss", dict(logit=logit, tok=lm_tok), dict(loss=loss, amax=amax))

    G = {}
    dlogit = o.softmax_ce_bwd(logit, lm_tok, scale)
    rec("softmax_ce_bwd", "loss", dict(logit=logit, tok=lm_tok, scale=scale), dict(dlogit=dlogit))
    G["lm_head"] = mm("lm_head.dW", 1, 0, dlogit, hn)
    dhn = mm("lm_head.dx", 0, 0, dlogit, P["lm_head"])
    dstream, G["head_norm"] = norm_b("head_norm", stream, P["head_norm"], dhn, None)
    for l in range(L - 1, -1, -1):
        g = lambda n: P["l%d.%s" % (l, n)]
        w = "l%d." % l
        s = saved[l]
        dx1 = dstream.copy()
        G[w + "down"] = mm(w + "down.dW", 1, 0, dstream, s["h"])
        dh = mm(w + "down.dx", 0, 0, dstream, g("down"))
        dgate, dup = o.silu_gate_bwd(s["gate"], s["up"], dh)
        rec("silu_gate_bwd", w + "silu_gate", dict(g=s["gate"], u=s["up"], dh=dh), dict(dg=dgate, du=dup))
        G[w + "gate"] = mm(w + "gate.dW", 1, 0, dgate, s["post"])
        dpost = mm(w + "gate.dx", 0, 0, dgate, g("gate"))
        G[w + "up"] = mm(w + "up.dW", 1, 0, dup, s["post"])
        dpost = mm(w + "up.dx", 0, 0, dup, g("up"), 1.0, 1.0, dpost)
        dx1, G[w + "post_norm"] = norm_b(w + "post_norm", s["x1"], g("post_norm"), dpost, dx1)
        dx0 = dx1.copy()
        G[w + "o"] = mm(w + "o.dW", 1, 0, dx1, s["attn"])
        dattn = mm(w + "o.dx", 0, 0, dx1, g("o"))
        dv = bmm(w + "pv.dB", 1, 0, S, Dh, S, 1.0, s["p16"], lds, S, dattn, ld, Dh, (S, D), ld, Dh, 3)
        dp16 = bmm(w + "pv.dA", 0, 1, S, S, Dh, 1.0, dattn, ld, Dh, s["v"], ld, Dh, (S, H, S), lds, S, 1)
        ds16 = o.causal_softmax_bwd(s["s16"], dp16)
        rec("causal_softmax_bwd", w + "softmax", dict(s16=s["s16"], dp16=dp16), dict(ds16=ds16))
        dkr = bmm(w + "qk.dB", 1, 0, S, Dh, S, alpha, ds16, lds, S, s["qr"], ld, Dh, (S, D), ld, Dh, 3)
        dqr = bmm(w + "qk.dA", 0, 0, S, Dh, S, alpha, ds16, lds, S, s["kr"], ld, Dh, (S, D), ld, Dh, 2)
        sh = lambda a: a.reshape(S, H, Dh)
        rec("attention_bwd", w + "attention",
            dict(q=sh(s["qr"]), k=sh(s["kr"]), v=sh(s["v"]), o=sh(s["attn"]), dO=sh(dattn), alpha=alpha),
            dict(dq=sh(dqr), dk=sh(dkr), dv=sh(dv)))
        G[w + "v"] = mm(w + "v.dW", 1, 0, dv, s["pre"])
        dpre = mm(w + "v.dx", 0, 0, dv, g("v"))
        dk = rope_b(w + "k", dkr)
        G[w + "k"] = mm(w + "k.dW", 1, 0, dk, s["pre"])
        dpre = mm(w + "k.dx", 0, 0, dk, g("k"), 1.0, 1.0, dpre)
        dq = rope_b(w + "q", dqr)
        G[w + "q"] = mm(w + "q.dW", 1, 0, dq, s["pre"])
        dpre = mm(w + "q.dx", 0, 0, dq, g("q"), 1.0, 1.0, dpre)
        dstream, G[w + "pre_norm"] = norm_b(w + "pre_norm", s["x0"], g("pre_norm"), dpre, dx0)
    G["embed"] = o.embed_bwd(V, tok, dstream)
    rec("embed_bwd", "embed", dict(V=V, tok=tok, dy=dstream), dict(dW=G["embed"]))
    return calls, loss, G
