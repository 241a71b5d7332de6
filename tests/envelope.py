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

The set of restatements is frozen (tests/test_oracle_restatements.py pins each mode against fp64
arithmetic and fails if the set changes): a maximum over pairs grows with every member, so a bar
that may be widened at will is no bar.  Three more conditions keep it honest:
  * an absolute cap beside it (ABS_CAP): whatever the restatements do, no gradient tensor may be
    further than 2e-3 relative L2 from the oracle's default run;
  * the device must not be an outlier of the family: its mean distance to the restatements may not
    exceed the largest mean distance one restatement has to the others (OUTLIER_SLACK covers the
    sampling noise of twelve points);
  * the table printed shows the device's distance to every restatement, so that a device result
    that sits next to one particular order (or far from all of them) is visible.
"""
import itertools

import numpy as np

from tests.util import max_rel, rel_l2

ABS_CAP = 2e-3
OUTLIER_SLACK = 1.02
LOSS_ABS_CAP = 2e-4


class Envelope(dict):
    """{tensor: (rel_l2, max_rel)} plus the runs it was measured from (restatement -> {tensor: grad}) and the
    same pair of figures for the per-position loss."""
    runs = None
    loss = None
    loss_to_default = None


def order_envelope(oracle, cfg, flat, tok, lm_tok, scale, grad_cached=None, count=None):
    """Returns (runs: restatement -> {tensor: grad}, env: Envelope); count: only the first `count`
    restatements (large shapes)."""
    runs, losses = {}, {}
    try:
        for name in list(oracle.RESTATEMENTS)[:count]:
            oracle.set_restatement(name)
            out = oracle.llama_step(cfg, flat, tok, lm_tok, scale, grad_cached=grad_cached)
            runs[name] = oracle.split_params(cfg, out["grad"])
            losses[name] = np.asarray(out["loss"], np.float64)
    finally:
        oracle.set_restatement("ascending")
    env = Envelope()
    env.runs = runs
    pairs = list(itertools.combinations(runs, 2))
    env.loss = (max(rel_l2(losses[a], losses[b]) for a, b in pairs),
                max(max_rel(losses[a], losses[b]) for a, b in pairs))
    env.loss_to_default = {n: rel_l2(losses[n], losses["ascending"]) for n in losses if n != "ascending"}
    for t in runs["ascending"]:
        env[t] = (max(rel_l2(runs[a][t], runs[b][t]) for a, b in pairs),
                  max(max_rel(runs[a][t], runs[b][t]) for a, b in pairs))
    return runs, env


def family_distances(got, runs):
    """Per tensor: (device's distance to each restatement {name: d}, each restatement's mean distance to
    the other restatements {name: d})."""
    names = list(runs)
    out = {}
    for t, g in got.items():
        dev = {n: rel_l2(g, runs[n][t]) for n in names}
        pair = {(a, b): rel_l2(runs[a][t], runs[b][t]) for a, b in itertools.combinations(names, 2)}
        mean = {n: sum(d for p, d in pair.items() if n in p) / (len(names) - 1) for n in names}
        out[t] = (dev, mean)
    return out


def assert_inside_envelope(got, want, env, tag, verbose=True, abs_cap=ABS_CAP):
    """got, want: {tensor: array}; asserts rel_l2 and max_rel of got vs want <= the envelope per tensor
    (ratio <= 1.0), rel_l2 <= abs_cap, and, when the envelope carries its runs, that the device is not
    an outlier of the family; prints the tables."""
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
    fam = family_distances(got, env.runs) if getattr(env, "runs", None) else {}
    if fam and verbose:
        names = list(env.runs)
        print("%s: rel_l2 x 1e3 of the device to each restatement | mean of the device | largest and smallest "
              "mean of a restatement to the others" % tag)
        print("  %-14s %s" % ("", " ".join("%5d" % i for i in range(len(names)))))
        for t, (dev, mean) in fam.items():
            dm = sum(dev.values()) / len(dev)
            print("  %-14s %s | %.3f | %.3f %.3f" % (t, " ".join("%5.2f" % (1e3 * dev[n]) for n in names), 1e3 * dm,
                                                   1e3 * max(mean.values()), 1e3 * min(mean.values())))
        print("  restatements: " + ", ".join("%d=%s" % (i, n) for i, n in enumerate(names)), flush=True)
    for t, e2, f2, r, em, fm in rows:
        assert e2 <= f2, "%s:%s rel_l2 %.3e outside the envelope %.3e" % (tag, t, e2, f2)
        assert e2 <= abs_cap, "%s:%s rel_l2 %.3e above the absolute cap %.1e" % (tag, t, e2, abs_cap)
        assert em <= max(fm, 2e-2), "%s:%s max_rel %.3e outside the envelope %.3e" % (tag, t, em, fm)
    for t, (dev, mean) in fam.items():
        dm = sum(dev.values()) / len(dev)
        assert dm <= OUTLIER_SLACK * max(mean.values()), \
            "%s:%s the device is an outlier: mean distance %.3e to the restatements, theirs at most %.3e" % (
                tag, t, dm, max(mean.values()))
    return worst


def assert_loss_inside_envelope(loss, want, env, tag):
    """The per-position loss of a composed run is the end of the same chain of f16-rounded products as the
    gradients: at the 3B shapes the restatements' own losses are 0.9e-4 .. 1.4e-4 relative L2 from the default
    one after a single layer.  So it is held to the largest distance between two restatements, and to the
    absolute cap LOSS_ABS_CAP beside it; the loss thunk by itself is held to 1e-5 on the oracle's logits
    (tests/test_gpu_full_shapes.py::test_lm_head_and_cross_entropy_full_shape, tests/test_gpu_teacher.py)."""
    e2, em = rel_l2(loss, want), max_rel(loss, want)
    f2, fm = env.loss
    print("%s: loss rel_l2 %.3e  envelope %.3e  ratio %.2f   max_rel %.3e  envelope %.3e; restatements to the "
          "default one: %s" % (tag, e2, f2, e2 / f2, em, fm,
                               " ".join("%.2e" % v for v in env.loss_to_default.values())), flush=True)
    assert e2 <= f2, "%s: loss rel_l2 %.3e outside the envelope %.3e" % (tag, e2, f2)
    assert e2 <= LOSS_ABS_CAP, "%s: loss rel_l2 %.3e above the absolute cap %.1e" % (tag, e2, LOSS_ABS_CAP)
    assert em <= max(fm, 1e-3), "%s: loss max_rel %.3e outside the envelope %.3e" % (tag, em, fm)
    return e2
