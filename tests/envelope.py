"""The summation-order envelope of the composed cycle (test helper).

The reference fixes "f16 products, fp32 accumulate" for its GEMMs but not the order of the fp32
sums (cuBLAS picks it), nor the association order of its f32 reductions (Futhark's), nor the last
ulp of exp / log (libm's).  A chain of f16-rounded GEMMs turns any such change into independent f16
rounding flips which later layers re-amplify, so two correct implementations differ by about 1e-3
relative L2 after two layers.  The envelope is measured, not assumed: the oracle runs the same cycle
as twelve restatements (oracle.RESTATEMENTS: eight GEMM summation orders, some of them also with
reductions summed in f32 and / or correctly rounded exp / log) and, per gradient tensor, the largest
distance between any two of them is the bar for one more implementation (the device) against the
oracle's default run.
"""
import itertools

from tests.util import max_rel, rel_l2


def order_envelope(oracle, cfg, flat, tok, lm_tok, scale, grad_cached=None, count=None):
    """Returns (runs: restatement -> {tensor: grad}, env: {tensor: (rel_l2, max_rel)}); count: only the
    first `count` restatements (large shapes)."""
    runs = {}
    try:
        for name in list(oracle.RESTATEMENTS)[:count]:
            oracle.set_restatement(name)
            out = oracle.llama_step(cfg, flat, tok, lm_tok, scale, grad_cached=grad_cached)
            runs[name] = oracle.split_params(cfg, out["grad"])
    finally:
        oracle.set_restatement("ascending")
    env = {}
    for t in runs["ascending"]:
        pairs = list(itertools.combinations(runs, 2))
        env[t] = (max(rel_l2(runs[a][t], runs[b][t]) for a, b in pairs),
                  max(max_rel(runs[a][t], runs[b][t]) for a, b in pairs))
    return runs, env


def assert_inside_envelope(got, want, env, tag, verbose=True):
    """got, want: {tensor: array}; asserts rel_l2 and max_rel of got vs want <= the envelope per tensor
    (ratio <= 1.0) and prints the table."""
    worst = 0.0
    rows = []
    for t, g in got.items():
        e2, em = rel_l2(g, want[t]), max_rel(g, want[t])
        f2, fm = env[t]
        rows.append((t, e2, f2, e2 / f2, em, fm))
        worst = max(worst, e2 / f2)
    if verbose:
        print("%s: device vs oracle against the summation-order envelope" % tag)
        for t, e2, f2, r, em, fm in rows:
            print("  %-14s rel_l2 %.3e  envelope %.3e  ratio %.2f   max_rel %.3e  envelope %.3e" % (t, e2, f2, r, em, fm))
        print("%s: worst ratio %.2f" % (tag, worst), flush=True)
    for t, e2, f2, r, em, fm in rows:
        assert e2 <= f2, "%s:%s rel_l2 %.3e outside the envelope %.3e" % (tag, t, e2, f2)
        assert em <= max(fm, 2e-2), "%s:%s max_rel %.3e outside the envelope %.3e" % (tag, t, em, fm)
    return worst
