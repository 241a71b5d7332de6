#!/usr/bin/env python3
"""bench.py -- fwd + loss + full-gradient bwd tokens/sec of the OpenLLaMA-3B-shaped fp16 step
on one MI355X, with the roofline of the dominant kernel and the CPU port timed beside it.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--pool-gb G] [--no-cpu-baseline]
    python bench.py --workload adjoints      # HBM-bound adjoint kernels at 3B shapes
    python bench.py --workload gemm          # every GEMM shape of the step, standalone
    python bench.py --workload digests       # NaN counts + abs-log2 histograms of all parameters and gradients

Prints ONE JSON line on stdout.  A step = reset + stage + vadd_vjp + compile + resume of
the 26-layer cycle (the reference's per-cycle control flow), inputs resident on the device
except the 3 small input cells (tokens, labels, loss scale: 16 KiB) that are put every step.
"""
import argparse
import json
import os
import re
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

LLAMA_3B = dict(S=2048, D=3200, H=32, Dh=100, F=8640, V=32000, L=26, eps=1e-6)
PEAK_MFMA_F16_TFLOPS = 2500.0      # MI355X dense fp16 MFMA
PEAK_HBM_GBS = 8000.0              # MI355X HBM3E
EVENT_STRIDE = 17                  # timed region: 1 in 17 launches of the dominant kernel carries events (a pair
                                   # costs about 17 us of stream time, two gaps in the kernel trace; at 1 in 5 that
                                   # was 0.55 ms of a 50 ms step)


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def synth_params(model, seed=0, std=0.02):
    """Seeded synthetic weights ~N(0, std) (norm weights ~N(1, std)): one 2^26-element normal
    block, read at a tensor-dependent offset with wrap-around (drawing 3.4e9 fresh normals on
    the host would take minutes and changes nothing that is measured)."""
    r = np.random.default_rng(seed)
    n = 1 << 26
    block = (r.standard_normal(n, dtype=np.float32) * std).astype(np.float16)
    off = 0
    for i, (name, shape) in enumerate(model.params):
        cnt = int(np.prod(shape))
        idx0 = (off * 7919) % n
        if idx0 + cnt <= n:
            w = block[idx0:idx0 + cnt]
        else:
            reps = (idx0 + cnt + n - 1) // n
            w = np.tile(block, reps)[idx0:idx0 + cnt]
        w = w.reshape(shape)
        if name.endswith("norm"):
            w = (w.astype(np.float32) + 1.0).astype(np.float16)
        model.put_param(i, w)
        off += cnt


def synth_inputs(cfg, seed=1, grad_scale=1024.0):
    r = np.random.default_rng(seed)
    tok = r.integers(0, cfg["V"], cfg["S"]).astype(np.uint16)
    lm_tok = np.concatenate([tok[1:], tok[:1]]).astype(np.uint16)
    scale = np.full(cfg["S"], grad_scale / (cfg["S"] - 1), np.float32)   # train.rs:521-530
    scale[0] = 0.0
    return tok, lm_tok, scale


# L2-miss traffic per launch of the GEMM kernels at the step's shapes: measured, not assumed, and tied to
# the kernels it was measured on.  cacti_amd/gemm_traffic.json is written by `python -m cacti_amd.gemm_traffic`
# from two rocprofv3 --pmc passes (FETCH_SIZE, WRITE_SIZE) over `bench.py --workload gemm-traffic` and
# records the hash of csrc/gemm_mfma.hip it was taken on; with any other build of the kernels the roofline
# line carries "traffic": null instead of figures that no longer describe what runs.
def _traffic_table():
    from cacti_amd import gemm_traffic
    return gemm_traffic.load_current()


def gemm_traffic_bytes(label, table):
    """Bytes per launch leaving the L2s for the product of a timing label, or None if not measured."""
    if not table:
        return None
    ent = table.get(label)
    return None if ent is None else float(ent["bytes"])


# "...]x3": three products of that shape staged as one thunk and launched together
GEMM_RE = re.compile(r"^(block_matmul|matmul)\[([NT])([NT]),(\d+)x(\d+)x(\d+)x(\d+)(,acc)?\](?:x(\d+))?$")


def gemm_group(label):
    m = GEMM_RE.match(label)
    return int(m.group(9) or 1) if m else 1


def gemm_flops(label):
    m = GEMM_RE.match(label)
    if not m:
        return None
    H, M, N, K = (int(m.group(i)) for i in (4, 5, 6, 7))
    return 2.0 * H * M * N * K * gemm_group(label)


N_CUS = 256


def attention_flops(label, cfg):
    """Algorithmic flops of the fused attention thunks: the causal half of Q K^T and P V in the
    forward pass (2 products of S^2/2 x Dh per head), of dV, dP, dQ and dK in the adjoint (4); what the
    kernels recompute (Q K^T again in both passes of the forward kernel and in both adjoint kernels) is
    not counted."""
    per = 2.0 * cfg["H"] * (cfg["S"] * (cfg["S"] + 1) // 2) * cfg["Dh"]
    return {"attention": 2 * per, "attention_bwd": 4 * per}.get(label)


def gemm_dims(label):
    m = GEMM_RE.match(label)
    return (m.group(2) == "T", m.group(3) == "T") + tuple(int(m.group(i)) for i in (4, 5, 6, 7))


def plan_tokens_product(M, N):
    """Mirror of plan_tokens_product in csrc/gemm_mfma.hip: (tile, columns of the first launch)."""
    best, best_cost = (4, N), None
    for tile, bn, round_cost in ((4, 128, 32768), (5, 256, 54613)):
        tiles_m, tiles_n = (M + 255) // 256, (N + bn - 1) // bn
        total = tiles_m * tiles_n
        full = total // N_CUS
        cols_main = full * N_CUS // tiles_m
        rest = tiles_m * (tiles_n - cols_main)
        if full >= 1 and cols_main < tiles_n and rest * bn * 4 <= N_CUS * 128:
            cost, main_cols = full * round_cost + 12288, cols_main * bn
        else:
            cost, main_cols = -(-total // N_CUS) * round_cost, N
        if best_cost is None or cost < best_cost:
            best, best_cost = (tile, main_cols), cost
    return best


TILE_ARGS = {0: "128, 128, 2, 2, 8, false, 2, 2, false", 4: "256, 128, 4, 2, 8, false, 1, 3, true",
             5: "256, 256, 2, 4, 8, false, 1, 2, true", 6: "256, 192, 4, 2, 8, false, 1, 2, true"}


def kernel_symbol(label):
    """Name of the HIP kernel instantiation a dense GEMM label runs on (its first launch), as
    rocprofv3 prints it.  The tile choice mirrors gemm_mfma_launch for 16-byte aligned operands
    and K % 64 == 0: with an output of at least 1024 x 1024 and one block, A not transposed runs
    256 x 128 or 256 x 256 / 8 waves by plan_tokens_product, A transposed 256 x 256 / 8 waves from
    2048 x 2048 outputs on (256 x 192 where that fills the CUs markedly better), all with
    direct-to-LDS loads; everything else 128 x 128 / 4 waves through registers."""
    ta, tb, H, M, N, K = gemm_dims(label)
    tile = 0
    if H == 1 and M >= 1024 and N >= 1024:
        if not ta:
            tile = plan_tokens_product(M, N)[0]
        elif M >= 2048 and N >= 2048:
            fill = lambda t: t / (-(-t // N_CUS) * N_CUS)
            tiles256 = ((M + 255) // 256) * ((N + 255) // 256)
            tiles192 = ((M + 255) // 256) * ((N + 191) // 192)
            tile = 6 if fill(tiles192) > 1.2 * fill(tiles256) else 5
    return "gemm_mfma_kernel<%s, %s, %s>" % (str(ta).lower(), str(tb).lower(), TILE_ARGS[tile])


def is_split(label):
    """True if the thunk issues two kernels (the columns beyond the full rounds of its tiles go to
    a second launch of 64 x 64 tiles): its event pair then brackets both, so it is left out of a
    single kernel's roofline sample."""
    ta, tb, H, M, N, K = gemm_dims(label)
    if gemm_group(label) > 1:                              # a grouped thunk: never one launch of one product
        return True
    if ta or H != 1 or M < 1024 or N < 1024 or K % 64:
        return False
    return plan_tokens_product(M, N)[1] < N


def label_prefix(label):
    """'matmul[TN' of 'matmul[TN,1x8640x3200x2048]': what the runtime's timing filter matches."""
    return label.split(",")[0]


CPU_SAMPLE_LAYERS = 3


def cpu_baseline(cfg):
    """The CPU port (the oracle) on a bounded sample of the same workload (about 10 s of CPU
    work): the LM head + loss alone and with 3 decoder layers at full shapes, forward + backward,
    extrapolated to 26 layers."""
    from oracle import oracle as o
    from tests.llama_ref import make_inputs
    times = {}
    for L in (0, CPU_SAMPLE_LAYERS):
        c = dict(cfg, L=L)
        ocfg, flat, tok, lm_tok, scale = make_inputs(c, seed=0, norm_mean=1.0, grad_scale=1024.0)
        t0 = time.time()
        o.llama_step(ocfg, flat, tok, lm_tok, scale)
        times[L] = time.time() - t0
        log("cpu_baseline: oracle L=%d fwd+bwd %.2f s" % (L, times[L]))
    layer = max(times[CPU_SAMPLE_LAYERS] - times[0], 1e-9) / CPU_SAMPLE_LAYERS
    full = times[0] + cfg["L"] * layer
    return {"value": cfg["S"] / full, "unit": "tokens/s", "cores": o.num_threads(), "kind": "port",
            "sample": "oracle fwd+bwd of %d of %d layers (%.2f s each) and of embedding+LM head+loss "
                      "(%.2f s) at full shapes, S=%d; step time extrapolated as head + %d x layer"
                      % (CPU_SAMPLE_LAYERS, cfg["L"], layer, times[0], cfg["S"], cfg["L"])}


# gradients read back after the capped and the uncapped leg and compared bit for bit (the layers are
# clipped to the model's depth): the first and last layers, one of every kind of tensor
CAPPED_PROBES = ["embed", "l0.q", "l0.pre_norm", "l3.k", "l7.down", "l12.up", "l18.gate", "l25.v", "l25.o",
                 "l25.post_norm", "head_norm", "lm_head"]


def probe_grads(model, cfg):
    """{name: f16 gradient} of CAPPED_PROBES for this model."""
    idx = {name: i for i, (name, _) in enumerate(model.params)}
    out = {}
    for n in CAPPED_PROBES:
        if n.startswith("l") and "." in n and n[1].isdigit():
            layer, rest = n.split(".", 1)
            n = "l%d.%s" % (min(int(layer[1:]), cfg["L"] - 1), rest)
        out[n] = model.grad(idx[n])
    return out


CAPPED_POOL_BYTES = 16 << 30       # the reference's 16 GiB card (examples/open_llama_3b_train.rs runs on one)
CAPPED_WARMUP = 6                  # the spill plan of a cycle follows the cycles before it: a few to settle


def run_capped(cfg, args):
    """The same step on a device pool capped at 16 GiB, so that it has to spill to page-locked host
    memory: K timed steps after its own warmup.  Returns the record, the loss and the probe gradients,
    which the caller compares bit for bit with the uncapped run's.  (It runs before the uncapped leg: a 16 GiB pool
    allocated after the uncapped leg's pool of 90 % of the device has been freed measured 10 % slower.)"""
    import torch
    from cacti_amd.runtime import Ctx, Llama
    ctx = Ctx(0, CAPPED_POOL_BYTES, True)
    model = Llama(ctx, **cfg)
    synth_params(model)
    tok, lm_tok, scale = synth_inputs(cfg)
    for _ in range(max(args.warmup, CAPPED_WARMUP)):
        model.step(tok, lm_tok, scale, want_loss=False)
    ctx.sync()
    torch.cuda.synchronize()
    st0 = ctx.stats()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        model.step(tok, lm_tok, scale, want_loss=False)
    ctx.sync()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    st1 = ctx.stats()
    loss = model.step(tok, lm_tok, scale)
    grads = probe_grads(model, cfg)
    model.close()
    ctx.close()
    per = lambda k: (st1[k] - st0[k]) / args.steps
    log("capped at %.0f GiB: %.2f ms/step, %.0f evictions, %.2f GB down, %.2f GB up per step"
        % (CAPPED_POOL_BYTES / 2 ** 30, dt / args.steps * 1e3, per("n_evict"), per("bytes_d2h") / 1e9, per("bytes_h2d") / 1e9))
    return {"pool_cap_bytes": CAPPED_POOL_BYTES, "ms_per_step": dt / args.steps * 1e3,
            "tokens_per_s": cfg["S"] * args.steps / dt, "evictions": per("n_evict"),
            "d2h_bytes": per("bytes_d2h"), "h2d_bytes": per("bytes_h2d"), "pool_peak_bytes": st1["pool_peak"],
            "steps": args.steps, "warmup": max(args.warmup, CAPPED_WARMUP)}, loss, grads


def run_step(args):
    import torch
    from cacti_amd.runtime import Ctx, Llama
    cfg = dict(LLAMA_3B)
    if args.layers is not None:
        cfg["L"] = args.layers
    pool = int(args.pool_gb * (1 << 30)) if args.pool_gb else 0
    # the same configuration on the reference's 16 GiB card: a second run, on a capped pool
    capped, capped_loss, capped_grads = (None, None, None) if pool or args.no_capped else run_capped(cfg, args)
    ctx = Ctx(0, pool, True)
    model = Llama(ctx, **cfg)
    t0 = time.time()
    synth_params(model)
    log("params staged on the host in %.1f s" % (time.time() - t0))
    tok, lm_tok, scale = synth_inputs(cfg)
    for _ in range(args.warmup):
        model.step(tok, lm_tok, scale, want_loss=False)
    ctx.sync()

    # survey (untimed): one step with an event pair around every launch gives the per-label
    # device times and names the dominant kernel.  An event pair costs a few microseconds of
    # stream time, ~10 % of the step when all ~1500 launches carry one, so the timed region
    # below keeps events only on the dominant kernel's launches.
    ctx.set_timing(0)
    ctx.set_timing_filter("")
    ctx.set_timing(2)
    n_survey = 2
    for _ in range(n_survey):
        model.step(tok, lm_tok, scale, want_loss=False)
    ctx.sync()
    rep = ctx.timing_report()
    by_sym = {}
    kernels = []
    for label, (cnt, tot_ms) in sorted(rep.items(), key=lambda kv: -kv[1][1]):
        fl = gemm_flops(label)
        sec = tot_ms / cnt * 1e-3
        ent = {"label": label, "launches_per_step": cnt / n_survey, "avg_us": sec * 1e6,
               "total_ms_per_step": tot_ms / n_survey}
        # every entry against the roof that bounds it: the products (attention included) by
        # their algorithmic flops against dense fp16 MFMA, everything else by its operand
        # bytes (each input read once, each output written once) against HBM
        ent["bytes"] = ctx.operand_bytes.get(label, 0)
        afl = attention_flops(label, cfg) if fl is None else fl
        if afl is not None:
            ent.update(bound="mfma", flops=afl, tflops=afl / sec / 1e12, frac=afl / sec / 1e12 / PEAK_MFMA_F16_TFLOPS)
        else:
            ent.update(bound="hbm", GBs=ent["bytes"] / sec / 1e9, frac=ent["bytes"] / sec / 1e9 / PEAK_HBM_GBS)
        if fl is not None:
            if label.startswith("matmul") and not is_split(label):     # one thunk = one launch
                s_ = by_sym.setdefault(kernel_symbol(label), [0.0, set()])
                s_[0] += tot_ms
                s_[1].add(label_prefix(label))
        kernels.append(ent)
    dev_ms = sum(v[1] for v in rep.values()) / n_survey
    sym, (_, prefixes) = max(by_sym.items(), key=lambda kv: kv[1][0])
    assert len(prefixes) == 1, prefixes
    prefix = next(iter(prefixes))

    # timed region: exactly K steps, events around every EVENT_STRIDE-th launch of the dominant
    # kernel (the stride is coprime to the 6 such launches per layer and the 157 per step, so all
    # shapes are sampled)
    ctx.set_timing(0)
    ctx.set_timing_filter(prefix, EVENT_STRIDE)
    ctx.set_timing(2)
    torch.cuda.synchronize()
    st0 = ctx.stats()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        model.step(tok, lm_tok, scale, want_loss=False)
    ctx.sync()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    rep = ctx.timing_report()
    st1 = ctx.stats()
    ctx.set_timing(0)
    ctx.set_timing_filter("")
    loss = model.step(tok, lm_tok, scale)
    assert np.all(np.isfinite(loss)), "non-finite loss"
    grads = probe_grads(model, cfg) if capped is not None else None
    ms = dt / args.steps * 1e3
    tokens_s = cfg["S"] * args.steps / dt

    # the filter matches by label prefix: keep the launches that are exactly one launch of the
    # dominant kernel
    rep = {label: v for label, v in rep.items() if not is_split(label) and kernel_symbol(label) == sym}
    assert rep, "no sampled launch of %s" % sym
    fl = sum(gemm_flops(label) * cnt for label, (cnt, _) in rep.items())
    sec = sum(tot_ms for _, tot_ms in rep.values()) * 1e-3
    cnt = sum(c for c, _ in rep.values())
    achieved = fl / sec / 1e12
    table = _traffic_table()
    tr = [(gemm_traffic_bytes(label, table), c) for label, (c, _) in rep.items()]
    traffic = None if any(t is None for t, _ in tr) else sum(t * c for t, c in tr) / cnt
    roofline = {"bound": "mfma", "kernel": sym, "timed_launches": cnt,
                "avg_launch_us": sec / cnt * 1e6, "flops_per_launch": fl / cnt,
                "achieved": achieved, "peak": PEAK_MFMA_F16_TFLOPS, "unit": "TFLOP/s",
                "frac": achieved / PEAK_MFMA_F16_TFLOPS, "traffic": traffic,
                "traffic_note": ("bytes per launch leaving the L2s (MALL or HBM), mean over the timed launches; "
                                 "per-shape FETCH_SIZE / WRITE_SIZE readings of cacti_amd/gemm_traffic.json, "
                                 "taken on this build of the kernels") if traffic is not None else
                                "no counter readings for this build of the GEMM kernels (cacti_amd/gemm_traffic.json "
                                "was taken on another)"}
    out = {
        "metric": "fwd+bwd tokens/sec, 3B-shaped fp16 step, 1 GPU", "value": tokens_s,
        "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16", "data": "synthetic (seeded N(0,0.02) weights, uniform token ids)",
        "config": {"workload": "OpenLLaMA-3B-shaped full-gradient step: %d layers, hidden 3200, "
                               "32 heads x 100, ffn 8640, vocab 32000, batch 1, seq 2048, "
                               "fwd + softmax-CE loss + bwd" % cfg["L"],
                   "pool_cap_bytes": st1["pool_cap"], "pool_peak_bytes": st1["pool_peak"],
                   "spill_evictions_per_step": (st1["n_evict"] - st0["n_evict"]) / args.steps,
                   "spill_d2h_bytes_per_step": (st1["bytes_d2h"] - st0["bytes_d2h"]) / args.steps,
                   "spill_h2d_bytes_per_step": (st1["bytes_h2d"] - st0["bytes_h2d"]) / args.steps},
        "survey_device_ms_per_step": dev_ms,
        "roofline": roofline,
        "kernels": kernels[:24],
    }
    model.close()
    ctx.close()
    if capped is not None:
        assert np.array_equal(np.asarray(loss).view(np.uint32), np.asarray(capped_loss).view(np.uint32)), \
            "the capped run's loss differs from the uncapped run's"
        capped["loss_bit_identical"] = True
        for n, g in grads.items():
            assert np.array_equal(g.view(np.uint16), capped_grads[n].view(np.uint16)), \
                "gradient %s of the capped run differs from the uncapped run's" % n
        capped["grads_bit_identical"] = True
        capped["grads_compared"] = sorted(grads)
        out["config"]["capped"] = capped
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(LLAMA_3B)
    else:
        out["cpu_baseline"] = None
    return out


def time_launches(fn, stream_sync, n_warm=3, n_iter=50):
    """Median device time of fn(i) over n_iter launches, each between its own pair of events (torch
    events on the current stream, which is the stream cacti_amd.ops launches on).  The pair brackets
    everything fn(i) queues: a Python wrapper that allocates its outputs or issues a second small
    kernel (the weight-gradient finalize of the RMSNorm adjoint) is timed with that included; the
    kernel-trace summaries under profiles/ give the kernels alone."""
    import torch
    for i in range(n_warm):
        fn(i)
    torch.cuda.synchronize()
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(n_iter)]
    for i in range(n_iter):
        ev[i][0].record()
        fn(i)
        ev[i][1].record()
    torch.cuda.synchronize()
    return float(np.median([a.elapsed_time(b) for a, b in ev])) * 1e-3


def cpu_baseline_adjoints(N, D, H, Dh, F, V):
    """The CPU port (the oracle, OpenMP) on the same adjoint shapes, one call each after a warm-up call;
    value = GB/s of the SiLU-gate adjoint by its algorithmic bytes, like the GPU line."""
    from oracle import oracle as o
    r = np.random.default_rng(0)
    rn = lambda *s: r.standard_normal(s, dtype=np.float32).astype(np.float16)
    x, dy, w = rn(N, D), rn(N, D), rn(D)
    cos, sin = o.rope_tables(N, Dh)
    q = rn(N, H, Dh)
    g_, u_, dh_ = rn(N, F), rn(N, F), rn(N, F)
    rows = 256                                                    # softmax-CE: a slice of the rows, scaled up
    lg = (r.standard_normal((rows, V), dtype=np.float32) * 2).astype(np.float16)
    tok = r.integers(0, V, rows).astype(np.uint16)
    sc = np.full(rows, 1.0 / N, np.float32)
    jobs = {"rms_norm_bwd": (lambda: o.rmsnorm_bwd(x, w, 1e-6, dy), 1.0), "rope_bwd": (lambda: o.rope_bwd(q, cos, sin), 1.0),
            "silu_gate_bwd": (lambda: o.silu_gate_bwd(g_, u_, dh_), 1.0),
            "softmax_ce_bwd": (lambda: o.softmax_ce_bwd(lg, tok, sc), N / rows)}
    per = {}
    for name, (fn, scale) in jobs.items():
        fn()
        t0 = time.time()
        fn()
        per[name] = (time.time() - t0) * scale * 1e6
        log("cpu_baseline: oracle %-16s %10.0f us" % (name, per[name]))
    return {"value": 5 * 2 * N * F / (per["silu_gate_bwd"] * 1e-6) / 1e9, "unit": "GB/s", "cores": o.num_threads(), "kind": "port",
            "sample": "oracle, one call per kernel at the full shapes (softmax-CE: %d of %d rows, scaled)" % (rows, N),
            "per_kernel_us": per}


def run_adjoints(args):
    """The memory-bound adjoint kernels at 3B shapes; buffers rotate over > 256 MB so every launch
    reads HBM, not the Infinity Cache."""
    import torch
    from cacti_amd import ops
    N, D, H, Dh, F, V = 2048, 3200, 32, 100, 8640, 32000
    g = torch.Generator(device="cuda").manual_seed(0)

    def rn(*shape, std=1.0):
        return (torch.randn(*shape, device="cuda", generator=g) * std).half()

    res = []

    def add(name, sec, nbytes):
        res.append({"kernel": name, "us": sec * 1e6, "algorithmic_bytes": nbytes,
                    "achieved_GBs": nbytes / sec / 1e9, "frac_of_8TBs": nbytes / sec / 1e9 / PEAK_HBM_GBS})
        log("%-22s %8.1f us  %7.1f GB/s  (%.1f%% of 8 TB/s)" % (name, sec * 1e6, nbytes / sec / 1e9,
                                                             100 * nbytes / sec / 1e9 / PEAK_HBM_GBS))

    R = 8
    xs, dys, dxs = [rn(N, D) for _ in range(R)], [rn(N, D) for _ in range(R)], [rn(N, D) for _ in range(R)]
    w = rn(D)
    add("rms_norm_bwd", time_launches(lambda i: ops.rms_norm_bwd(xs[i % R], w, 1e-6, dys[i % R]), None),
        3 * 2 * N * D + 2 * 2 * D)
    # the form every layer norm of the step runs: dx accumulates (one more read of [N, D])
    add("rms_norm_bwd(dx+=)", time_launches(lambda i: ops.rms_norm_bwd(xs[i % R], w, 1e-6, dys[i % R], dxs[i % R], None), None),
        4 * 2 * N * D + 2 * 2 * D)
    add("rms_norm_fwd", time_launches(lambda i: ops.rms_norm_fwd(xs[i % R], w, 1e-6), None), 2 * 2 * N * D + 2 * D)
    cos, sin = ops.rope_tables(N, Dh)
    q = [rn(N, H, Dh) for _ in range(12)]
    add("rope_bwd", time_launches(lambda i: ops.rope_bwd(q[i % 12], cos, sin), None), 2 * 2 * N * H * Dh + 2 * 2 * N * Dh)
    add("rope_fwd", time_launches(lambda i: ops.rope_fwd(q[i % 12], cos, sin), None), 2 * 2 * N * H * Dh + 2 * 2 * N * Dh)
    del xs, dys, dxs, q
    R = 3
    gs, us, dhs = [rn(N, F) for _ in range(R)], [rn(N, F) for _ in range(R)], [rn(N, F) for _ in range(R)]
    add("silu_gate_bwd", time_launches(lambda i: ops.silu_gate_bwd(gs[i % R], us[i % R], dhs[i % R]), None), 5 * 2 * N * F)
    add("silu_gate_fwd", time_launches(lambda i: ops.silu_gate_fwd(gs[i % R], us[i % R]), None), 3 * 2 * N * F)
    del gs, us, dhs
    lg = [rn(N, V, std=2.0) for _ in range(3)]
    tok = torch.randint(0, V, (N,), device="cuda").to(torch.int16)
    sc = torch.full((N,), 1.0 / N, device="cuda")
    add("softmax_ce_bwd", time_launches(lambda i: ops.softmax_ce_bwd(lg[i % 3], tok, sc), None), 2 * 2 * N * V)
    # through the C entry point with outputs allocated once: the Python wrapper reads the token-range
    # status back after every call, which would time a host synchronisation instead of the kernel
    from cacti_amd import ffi
    ce_loss = torch.empty(N, device="cuda")
    ce_amax = torch.empty(N, dtype=torch.int16, device="cuda")
    ce_stat = torch.zeros(1, dtype=torch.int32, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    add("softmax_ce_fwd(loss)",
        time_launches(lambda i: ffi.call("cacti_hip_softmax_ce_fwd", N, V, lg[i % 3].data_ptr(), tok.data_ptr(), None,
                                         ce_loss.data_ptr(), ce_amax.data_ptr(), ce_stat.data_ptr(), st), None), 2 * N * V)
    assert int(ce_stat.item()) == 0
    del lg
    s16 = [rn(N, H, N) for _ in range(2)]
    dp = rn(N, H, N)
    # the kernels alone, into outputs allocated (and zeroed above the diagonal) once: the Python wrappers
    # zero-fill a fresh dense output per call.  Bytes: the causal half of each tensor, the diagonal included.
    p_out = [torch.zeros_like(s16[0]) for _ in range(2)]
    tri = 2 * H * (N * (N + 1) // 2)
    add("causal_softmax_fwd", time_launches(lambda i: ffi.call("cacti_hip_causal_softmax_fwd", N, H, s16[i % 2].data_ptr(),
                                                               p_out[i % 2].data_ptr(), st), None), 2 * tri)
    add("causal_softmax_bwd", time_launches(lambda i: ffi.call("cacti_hip_causal_softmax_bwd", N, H, s16[i % 2].data_ptr(),
                                                               dp.data_ptr(), p_out[i % 2].data_ptr(), st), None), 3 * tri)
    dom = max(res, key=lambda r: r["algorithmic_bytes"] if r["kernel"] == "silu_gate_bwd" else 0)
    cpu = None if args.no_cpu_baseline else cpu_baseline_adjoints(N, D, H, Dh, F, V)
    return {"metric": "HBM-bound adjoint kernels at OpenLLaMA-3B shapes", "value": dom["achieved_GBs"],
            "unit": "GB/s", "n_gpus": 1, "higher_is_better": True, "dtype": "f16",
            "config": {"workload": "adjoint microbench: RMSNorm [2048,3200], RoPE [2048,32,100], "
                                   "SiLU-gate [2048,8640], softmax-CE [2048,32000], causal softmax [2048,32,2048] (causal half)"},
            "roofline": {"bound": "hbm", "kernel": dom["kernel"], "achieved": dom["achieved_GBs"],
                         "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": dom["frac_of_8TBs"], "traffic": None},
            "cpu_baseline": cpu, "kernels": res}


def run_mfma_power(args):
    """The rate of MFMAs the device sustains over seconds (it is limited by power there, not by cycles): zero
    against random operands, the 32 x 32 x 16 against the 16 x 16 x 32 product, with and without the fragment
    reads of a 128 x 64 wave patch.  value = the sustained rate of the variant the large products of the step
    are built on (16 x 16 x 32, 6 fragment reads per k step, random operands)."""
    import torch
    from cacti_amd import ffi
    blocks, iters = 256, 100000
    out = torch.empty(blocks * 512, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    per_launch = 262144.0 * iters * 8 * blocks
    variants = [("32x32x16, zero operands, no LDS reads", 0, 0, 0), ("32x32x16, random operands, no LDS reads", 0, 0, 1),
                ("32x32x16, random, 4 fragment reads per k step", 0, 4, 1), ("32x32x16, random, 6 fragment reads per k step", 0, 6, 1),
                ("16x16x32, zero operands, no LDS reads", 1, 0, 0), ("16x16x32, random operands, no LDS reads", 1, 0, 1),
                ("16x16x32, random, 4 fragment reads per k step", 1, 4, 1), ("16x16x32, random, 6 fragment reads per k step", 1, 6, 1),
                ("32x32x16, random, 6 fragment reads per k step (again)", 0, 6, 1)]
    res = []
    for name, shape, reads, rnd in variants:
        ffi.call("cacti_hip_mfma_probe", shape, reads, rnd, blocks, 2000, 1, out.data_ptr(), st)
        torch.cuda.synchronize()
        t0, n = time.perf_counter(), 0
        while time.perf_counter() - t0 < args.sustain_probe:
            for _ in range(4):
                ffi.call("cacti_hip_mfma_probe", shape, reads, rnd, blocks, iters, 12345 + n, out.data_ptr(), st)
            torch.cuda.synchronize()
            n += 4
        dt = time.perf_counter() - t0
        res.append({"variant": name, "tflops": per_launch * n / dt / 1e12, "seconds": dt})
        log("%-56s %7.1f TFLOP/s sustained over %.1f s" % (name, res[-1]["tflops"], dt))
    key = res[7]["tflops"]
    return {"metric": "sustained MFMA rate, 16x16x32 f16 with fragment reads, random operands", "value": key,
            "unit": "TFLOP/s", "n_gpus": 1, "higher_is_better": True, "dtype": "f16",
            "config": {"workload": "MFMA-only probe, 256 workgroups of 8 waves, %.1f s per variant" % args.sustain_probe},
            "roofline": {"bound": "mfma", "achieved": key, "peak": PEAK_MFMA_F16_TFLOPS, "unit": "TFLOP/s",
                         "frac": key / PEAK_MFMA_F16_TFLOPS, "traffic": None},
            "cpu_baseline": None, "variants": res}


def run_gemm_traffic(args):
    """The dense products of the step, each launched gemm_traffic.LAUNCHES times in the order of
    gemm_traffic.STEP_PRODUCTS and nothing else: the dispatch sequence `python -m cacti_amd.gemm_traffic`
    expects in the counter files of a rocprofv3 --pmc run over this workload."""
    import torch
    from cacti_amd import gemm_traffic, ops
    g = torch.Generator(device="cuda").manual_seed(0)
    rn = lambda *s: (torch.randn(*s, device="cuda", generator=g) * 0.05).half()
    n = 0
    for label in gemm_traffic.STEP_PRODUCTS:
        ta, tb, _, M, N, K = gemm_dims(label)
        a = rn(K, M) if ta else rn(M, K)
        b = rn(N, K) if tb else rn(K, N)
        out = rn(M, N)
        beta = 1.0 if label.endswith(",acc]") else 0.0
        for _ in range(gemm_traffic.LAUNCHES):
            ops.gemm(a, b, ta, tb, 1.0, beta, out)
            n += 1
        torch.cuda.synchronize()
    return {"metric": "launches for the traffic counters", "value": n, "unit": "launches", "n_gpus": 1,
            "config": {"workload": "every dense product of the step x %d" % gemm_traffic.LAUNCHES}}


def run_gemm_step(args):
    """The dense products of one 26-layer step in the step's order, back to back and nothing else, so that
    the device sits in the thermal and power state of the step: time per pass and sustained TFLOP/s; with
    --yardstick the same sequence through the vendor library (torch.matmul / addmm -> hipBLASLt) beside it,
    a yardstick for what the device sustains on these shapes, no part of the product path."""
    import torch
    from cacti_amd import ops
    S, D, F, V, L = 2048, 3200, 8640, 32000, 26
    g = torch.Generator(device="cuda").manual_seed(0)
    rn = lambda *s, std=1.0: (torch.randn(*s, device="cuda", generator=g) * std).half()
    R = 3                                                   # operand sets in rotation
    x_d, x_f = [rn(S, D) for _ in range(R)], [rn(S, F) for _ in range(R)]
    w_dd, w_fd, w_df = [rn(D, D, std=0.02) for _ in range(R)], [rn(F, D, std=0.02) for _ in range(R)], \
        [rn(D, F, std=0.02) for _ in range(R)]
    o_d, o_f = torch.empty(S, D, device="cuda", dtype=torch.float16), torch.empty(S, F, device="cuda", dtype=torch.float16)
    g_dd, g_fd, g_df = (torch.empty(*s, device="cuda", dtype=torch.float16) for s in ((D, D), (F, D), (D, F)))
    x_v, w_vd, o_v, g_vd = rn(S, V, std=0.01), rn(V, D, std=0.02), torch.empty(S, V, device="cuda", dtype=torch.float16), \
        torch.empty(V, D, device="cuda", dtype=torch.float16)
    # (A, B, ta, tb, beta, out): the 21 products of a layer, then the 3 of the head
    def layer(i):
        a, f, wdd, wfd, wdf = x_d[i % R], x_f[i % R], w_dd[i % R], w_fd[i % R], w_df[i % R]
        fwd = [(a, wdd, 0, 1, 0.0, o_d)] * 4 + [(a, wfd, 0, 1, 0.0, o_f)] * 2 + [(f, wdf, 0, 1, 0.0, o_d)]
        bwd = [(a, wdf, 0, 0, 0.0, o_f), (a, f, 1, 0, 0.0, g_df),                        # down: dgrad, wgrad
               (f, wfd, 0, 0, 0.0, o_d), (f, a, 1, 0, 0.0, g_fd), (f, wfd, 0, 0, 1.0, o_d), (f, a, 1, 0, 0.0, g_fd),
               (a, wdd, 0, 0, 0.0, o_d), (a, a, 1, 0, 0.0, g_dd),                        # o
               (a, wdd, 0, 0, 0.0, o_d), (a, a, 1, 0, 0.0, g_dd), (a, wdd, 0, 0, 1.0, o_d), (a, a, 1, 0, 0.0, g_dd),
               (a, wdd, 0, 0, 1.0, o_d), (a, a, 1, 0, 0.0, g_dd)]
        return fwd, bwd
    head = [(x_d[0], w_vd, 0, 1, 0.0, o_v), (x_v, w_vd, 0, 0, 0.0, o_d), (x_v, x_d[0], 1, 0, 0.0, g_vd)]
    seq = [c for i in range(L) for c in layer(i)[0]] + head[:1] + head[1:] + [c for i in range(L) for c in layer(i)[1]]
    flops = 0.0
    for a, b, ta, tb, beta, out in seq:
        flops += 2.0 * out.shape[0] * out.shape[1] * (a.shape[0] if ta else a.shape[1])

    def ours():
        for a, b, ta, tb, beta, out in seq:
            ops.gemm(a, b, bool(ta), bool(tb), 1.0, beta, out)

    def library():
        for a, b, ta, tb, beta, out in seq:
            A_, B_ = (a.t() if ta else a), (b.t() if tb else b)
            if beta:
                torch.addmm(out, A_, B_, out=out)
            else:
                torch.matmul(A_, B_, out=out)

    def timed(fn, passes):
        fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(passes):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / passes

    passes = max(args.steps, 3)
    ms = timed(ours, passes)
    log("%d dense products of a step back to back: %.2f ms per pass, %.0f TFLOP/s sustained" % (len(seq), ms, flops / ms / 1e9))
    out = {"metric": "dense products of one step, back to back", "value": ms, "unit": "ms", "n_gpus": 1,
           "higher_is_better": False, "dtype": "f16", "tflops": flops / ms / 1e9, "products": len(seq), "passes": passes,
           "config": {"workload": "the %d dense products of the 26-layer 3B step in its order" % len(seq)}}
    if args.yardstick:
        yms = timed(library, passes)
        log("the same through the vendor library:            %.2f ms per pass, %.0f TFLOP/s sustained" % (yms, flops / yms / 1e9))
        out.update(library_ms=yms, library_tflops=flops / yms / 1e9)
    return out


def run_gemm(args):
    """Every GEMM shape of the step, standalone: TFLOP/s per shape."""
    import torch
    from cacti_amd import ops
    N, D, F, V, H, Dh = 2048, 3200, 8640, 32000, 32, 100
    g = torch.Generator(device="cuda").manual_seed(0)

    def rn(*shape, std=1.0):
        if args.operands == "zeros":                # no toggling in the matrix pipes: the device keeps its full clock
            return torch.zeros(*shape, device="cuda", dtype=torch.float16)
        return (torch.randn(*shape, device="cuda", generator=g) * std).half()

    res = []
    shapes = [("proj fwd NT", False, True, (N, D), (D, D)), ("proj dgrad NN", False, False, (N, D), (D, D)),
              ("proj wgrad TN", True, False, (N, D), (N, D)),
              ("ffn-up fwd NT", False, True, (N, D), (F, D)), ("ffn-up dgrad NN", False, False, (N, F), (F, D)),
              ("ffn-up wgrad TN", True, False, (N, F), (N, D)),
              ("ffn-down fwd NT", False, True, (N, F), (D, F)), ("ffn-down dgrad NN", False, False, (N, D), (D, F)),
              ("ffn-down wgrad TN", True, False, (N, D), (N, F)),
              ("head fwd NT", False, True, (N, D), (V, D)), ("head dgrad NN", False, False, (N, V), (V, D)),
              ("head wgrad TN", True, False, (N, V), (N, D))]
    for name, ta, tb, sa, sb in shapes:
        a, b = rn(*sa), rn(*sb, std=0.02)
        M, K = (sa[1], sa[0]) if ta else sa
        Nn = sb[0] if tb else sb[1]
        out = torch.empty(M, Nn, device="cuda", dtype=torch.float16)
        sec = time_launches(lambda i: ops.gemm(a, b, ta, tb, 1.0, 0.0, out), None)
        fl = 2.0 * M * Nn * K
        ent = {"shape": name, "M": M, "N": Nn, "K": K, "us": sec * 1e6, "tflops": fl / sec / 1e12}
        if args.yardstick:
            # the vendor library's GEMM (torch.matmul -> hipBLASLt) on the same operands: a yardstick for
            # what these shapes allow on this device, no part of the product path
            A_, B_ = (a.t() if ta else a), (b.t() if tb else b)
            ysec = time_launches(lambda i: torch.matmul(A_, B_, out=out), None)
            ent.update(library_us=ysec * 1e6, library_tflops=fl / ysec / 1e12)
        res.append(ent)
        log("%-18s M=%5d N=%5d K=%5d %9.1f us %7.1f TFLOP/s%s" % (name, M, Nn, K, sec * 1e6, fl / sec / 1e12,
            "   library %9.1f us %7.1f TFLOP/s" % (ent["library_us"], ent["library_tflops"]) if args.yardstick else ""))
    if args.sustain > 0:
        # the largest product in a loop for that many seconds (sample the clocks from another shell
        # meanwhile): the rate a power-limited device sustains, against the burst above
        a, b = rn(N, D), rn(V, D, std=0.02)
        out = torch.empty(N, V, device="cuda", dtype=torch.float16)
        t_end, n, t0 = time.time() + args.sustain, 0, time.time()
        while time.time() < t_end:
            for _ in range(50):
                ops.gemm(a, b, False, True, 1.0, 0.0, out)
            torch.cuda.synchronize()
            n += 50
        dt = time.time() - t0
        res.append({"shape": "head fwd NT, sustained %d s" % args.sustain, "M": N, "N": V, "K": D,
                    "us": dt / n * 1e6, "tflops": 2.0 * N * V * D * n / dt / 1e12})
        log("head fwd NT sustained over %.0f s: %.1f us, %.1f TFLOP/s" % (dt, dt / n * 1e6, res[-1]["tflops"]))
    q, k, v = rn(N, H, Dh), rn(N, H, Dh), rn(N, H, Dh)
    sec = time_launches(lambda i: ops.block_matmul_qk(q, k, 0.1), None, n_iter=20)
    fl = 2.0 * H * N * N * Dh
    res.append({"shape": "attn QK^T (32 blocks)", "us": sec * 1e6, "tflops": fl / sec / 1e12})
    log("%-18s %9.1f us %7.1f TFLOP/s (dense)" % ("attn QK^T", sec * 1e6, fl / sec / 1e12))
    p = rn(N, H, N)
    sec = time_launches(lambda i: ops.block_matmul_pv(p, v), None, n_iter=20)
    res.append({"shape": "attn PV (32 blocks)", "us": sec * 1e6, "tflops": fl / sec / 1e12})
    log("%-18s %9.1f us %7.1f TFLOP/s (dense)" % ("attn PV", sec * 1e6, fl / sec / 1e12))
    best = max(r["tflops"] for r in res)
    return {"metric": "GEMM shapes of the 3B step, standalone", "value": best, "unit": "TFLOP/s",
            "n_gpus": 1, "higher_is_better": True, "dtype": "f16",
            "config": {"workload": "f16 GEMM, fp32 accumulate, f16 out"},
            "roofline": {"bound": "mfma", "achieved": best, "peak": PEAK_MFMA_F16_TFLOPS,
                         "unit": "TFLOP/s", "frac": best / PEAK_MFMA_F16_TFLOPS, "traffic": None},
            "kernels": res}


def run_attention(args):
    """The fused causal attention thunk of one layer at the 3B shape (32 heads x 100, 2048 positions),
    standalone through the C entry points with outputs and workspace allocated once: forward and adjoint,
    against dense fp16 MFMA by their algorithmic flops (attention_flops)."""
    import torch
    from cacti_amd import ffi
    cfg = LLAMA_3B
    S, H, Dh = cfg["S"], cfg["H"], cfg["Dh"]
    g = torch.Generator(device="cuda").manual_seed(0)
    R = 4                                                   # operand sets in rotation

    def rn():
        return [torch.randn(S, H, Dh, device="cuda", generator=g).half() for _ in range(R)]

    q, k, v, dO = rn(), rn(), rn(), rn()
    o, dq, dk, dv = (torch.empty(S, H, Dh, device="cuda", dtype=torch.float16) for _ in range(4))
    stats = torch.empty(ffi.lib().cacti_hip_attention_stats_bytes(S, H) // 4, device="cuda")
    ws_bytes = ffi.lib().cacti_hip_attention_bwd_workspace(S, H)
    ws = torch.empty(max(ws_bytes, 4) // 4, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    alpha = 1.0 / float(np.sqrt(np.float32(Dh)))
    ld = H * Dh

    def fwd(i):
        ffi.call("cacti_hip_attention_fwd", S, H, Dh, alpha, q[i % R].data_ptr(), k[i % R].data_ptr(), v[i % R].data_ptr(),
                 ld, o.data_ptr(), stats.data_ptr(), st)

    def bwd(i):
        ffi.call("cacti_hip_attention_bwd", S, H, Dh, alpha, q[0].data_ptr(), k[0].data_ptr(), v[0].data_ptr(),
                 o.data_ptr(), dO[i % R].data_ptr(), ld, stats.data_ptr(), dq.data_ptr(), 0, dk.data_ptr(), 0, dv.data_ptr(), 0,
                 ws.data_ptr(), ws_bytes, st)

    res = []
    t_f = time_launches(fwd, None)
    fwd(0)                                                  # the statistics and output of operand set 0 for the adjoint
    t_b = time_launches(bwd, None)
    tensor = S * H * Dh * 2
    for label, sec, nbytes in (("attention", t_f, 4 * tensor + stats.numel() * 4),
                               ("attention_bwd", t_b, 8 * tensor + stats.numel() * 4)):
        fl = attention_flops(label, cfg)
        res.append({"kernel": label, "us": sec * 1e6, "flops": fl, "bytes": nbytes, "tflops": fl / sec / 1e12,
                    "frac": fl / sec / 1e12 / PEAK_MFMA_F16_TFLOPS, "bound": "mfma"})
        log("%-14s %8.1f us  %6.1f TFLOP/s (algorithmic, %.1f%% of 2500)  operands %.1f MB"
            % (label, sec * 1e6, fl / sec / 1e12, 100 * res[-1]["frac"], nbytes / 1e6))
    tot = t_f + t_b
    cpu = None
    if not args.no_cpu_baseline:
        # the CPU port (the oracle's chain of separate thunks) on 4 of the 32 heads, scaled
        from oracle import oracle as o
        hs = 4
        qc, kc, vc, gc = (t[0][:, :hs].contiguous().cpu().numpy() for t in (q, k, v, dO))
        t0 = time.time()
        o.attention_fwd(qc, kc, vc, alpha)
        t1 = time.time()
        o.attention_bwd(qc, kc, vc, gc, alpha)
        t2 = time.time()
        cpu = {"value": ((t1 - t0) + (t2 - t1)) * H / hs * 1e6, "unit": "us", "cores": o.num_threads(), "kind": "port",
               "sample": "oracle attention_fwd + attention_bwd (dense, as the reference executes it) on %d of %d heads, "
                         "scaled: fwd %.0f us, bwd %.0f us" % (hs, H, (t1 - t0) * H / hs * 1e6, (t2 - t1) * H / hs * 1e6)}
        log("cpu_baseline: " + cpu["sample"])
    return {"metric": "fused causal attention of one layer, fwd + adjoint", "value": tot * 1e6, "unit": "us",
            "n_gpus": 1, "higher_is_better": False, "dtype": "f16",
            "config": {"workload": "causal attention, %d heads x %d, %d positions, one layer" % (H, Dh, S)},
            "roofline": {"bound": "mfma", "kernel": "attn_bwd (dq + dkv kernels)", "achieved": res[1]["tflops"],
                         "peak": PEAK_MFMA_F16_TFLOPS, "unit": "TFLOP/s", "frac": res[1]["frac"], "traffic": None},
            "cpu_baseline": cpu, "kernels": res}


def run_digests(args):
    """The numerical-health digests the reference's example takes every cycle: nan_count and
    abs_log2_hist8 of each of the 237 parameters and 237 gradients (2 x 6.85 GB of f16), after one
    step; value = bytes digested per second, the CPU port timed on the embedding alone."""
    import torch
    from cacti_amd.runtime import Ctx, Llama
    cfg = dict(LLAMA_3B)
    if args.layers is not None:
        cfg["L"] = args.layers
    ctx = Ctx(0, 0, True)
    model = Llama(ctx, **cfg)
    synth_params(model)
    tok, lm_tok, scale = synth_inputs(cfg)
    model.step(tok, lm_tok, scale, want_loss=False)
    for g in (True, False):
        model.digests(of_grads=g)
    ctx.sync()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        gh, gn = model.digests(of_grads=True)
        ph, pn = model.digests(of_grads=False)
    dt = (time.perf_counter() - t0) / args.steps
    nbytes = 2 * 2 * int(ph.sum())                       # every element is counted once per histogram
    assert int(gh.sum()) == int(ph.sum()) and int(gn.sum()) == 0 and int(pn.sum()) == 0
    out = {"metric": "numerical-health digests (nan_count + abs_log2_hist8) of all parameters and gradients",
           "value": nbytes / dt / 1e9, "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": 1,
           "ms_per_step": dt * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
           "dtype": "u16", "data": "synthetic (the benchmark step's parameters and gradients)",
           "config": {"workload": "2 x %d f16 tensors, %.2f GB each set, both digests of a set in one launch"
                                  % (len(model.params), int(ph.sum()) * 2 / 1e9)},
           "roofline": {"bound": "hbm", "achieved": nbytes / dt / 1e9, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                        "frac": nbytes / dt / 1e9 / PEAK_HBM_GBS, "traffic": None,
                        "note": "every tensor is read once; wall time of the two model-level calls "
                                "including their stream synchronisations and result copies"}}
    model.close()
    ctx.close()
    if not args.no_cpu_baseline:
        from oracle import oracle as o
        x = (np.random.default_rng(0).standard_normal((cfg["V"], cfg["D"])) * 0.02).astype(np.float16)
        t0 = time.time()
        o.abs_log2_hist8(x)
        o.nan_count(x)
        t = time.time() - t0
        out["cpu_baseline"] = {"value": x.nbytes / t / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
                               "sample": "oracle digests of one [32000, 3200] f16 tensor (%.2f s)" % t}
    else:
        out["cpu_baseline"] = None
    return out


def run_adamw(args):
    """One AdamW32 step of every parameter of the 3B model (the minibatch boundary of the reference's
    example, examples/open_llama_3b_train.rs:252-268, which it runs on the CPU): moment averages,
    master-weight update and the cast back to f16, one launch.  value = parameters updated per second;
    algorithmic bytes = 28 per parameter (read f16 grad + 3 f32 states, write 3 f32 states + f16 param)."""
    import torch
    from cacti_amd.runtime import Ctx, Llama
    cfg = dict(LLAMA_3B)
    if args.layers is not None:
        cfg["L"] = args.layers
    opt = dict(grad_scale=1024.0, lr=2.0e-5, wd=0.1, a1=0.1, a2=0.05, eps=1.0e-5)   # the example's AdamW32
    ctx = Ctx(0, 0, True)
    model = Llama(ctx, **cfg)
    synth_params(model)
    tok, lm_tok, scale = synth_inputs(cfg)
    model.step(tok, lm_tok, scale, want_loss=False)
    model.adamw_init()
    nparam = sum(int(np.prod(shp)) for _, shp in model.params)
    for it in range(1, args.warmup + 1):
        model.adamw_step(it, **opt)
    ctx.sync()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for it in range(args.warmup + 1, args.warmup + args.steps + 1):
        model.adamw_step(it, **opt)
    ctx.sync()
    dt = (time.perf_counter() - t0) / args.steps
    # property that holds at any size: the parameters are the f16 rounding of the master weights
    for i in (1, len(model.params) - 1):
        assert np.array_equal(model.param(i).view(np.uint16),
                              model.adamw_state(i, "master").astype(np.float16).view(np.uint16))
    out = {"metric": "AdamW32 step (moment averages, master update, cast to f16) over all parameters",
           "value": nparam / dt, "unit": "parameters/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
           "ms_per_step": dt * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
           "dtype": "f32", "data": "synthetic (the benchmark step's parameters and gradients)",
           "config": {"workload": "%d tensors, %.3f G parameters, one launch per step" % (len(model.params), nparam / 1e9)},
           "roofline": {"bound": "hbm", "achieved": 28.0 * nparam / dt / 1e9, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                        "frac": 28.0 * nparam / dt / 1e9 / PEAK_HBM_GBS, "traffic": None,
                        "note": "28 bytes per parameter; wall time of the calls, synchronised once at the end"}}
    model.close()
    ctx.close()
    if not args.no_cpu_baseline:
        from oracle import oracle as o
        r = np.random.default_rng(0)
        n = cfg["V"] * cfg["D"]
        g = (r.standard_normal(n, dtype=np.float32) * 0.3).astype(np.float16)
        a = np.zeros(n, np.float32); b = np.zeros(n, np.float32)
        w = r.standard_normal(n, dtype=np.float32) * 0.02
        sc = o.adamw32_scalars(2, **opt)
        p16 = np.empty(n, np.float16)
        o.lib().oracle_adamw32_step(o.i64(n), o.P(g), o.P(a), o.P(b), o.P(w), o.P(p16), o.P(sc))   # touch the pages
        t0 = time.time()
        reps = 3
        for _ in range(reps):
            o.lib().oracle_adamw32_step(o.i64(n), o.P(g), o.P(a), o.P(b), o.P(w), o.P(p16), o.P(sc))
        t = (time.time() - t0) / reps
        out["cpu_baseline"] = {"value": n / t, "unit": "parameters/s", "cores": o.num_threads(), "kind": "port",
                               "sample": "oracle AdamW32 step (four thunks) of one [32000, 3200] tensor, in place, "
                                         "%d repetitions of %.2f s" % (reps, t)}
    else:
        out["cpu_baseline"] = None
    return out


def run_ingest(args):
    """Weight ingest (src/util/safetensor.rs:45-160 + resume_put + set_lossy_cast): a bf16 safetensors
    checkpoint of the 3B model's embedding, first `--layers` (default 4) layers and LM head is written
    to a temporary directory, then opened, matched and stored into the f16 parameter cells through
    the device cast; value = checkpoint bytes per second from the page cache into device cells (the
    path crosses PCIe: it is bound by the host copy into the staging cell and the upload, not by HBM)."""
    import shutil
    import struct
    import tempfile
    import torch
    from cacti_amd import ingest
    from cacti_amd.runtime import Ctx, Llama
    from oracle import oracle as o
    cfg = dict(LLAMA_3B)
    cfg["L"] = args.layers if args.layers is not None else 4
    ctx = Ctx(0, 0, True)
    model = Llama(ctx, **cfg)
    keys = ["model.embed_tokens.weight"]
    for i in range(cfg["L"]):
        p = "model.layers.%d." % i
        keys += [p + "input_layernorm.weight", p + "self_attn.q_proj.weight", p + "self_attn.k_proj.weight",
                 p + "self_attn.v_proj.weight", p + "self_attn.o_proj.weight", p + "post_attention_layernorm.weight",
                 p + "mlp.gate_proj.weight", p + "mlp.up_proj.weight", p + "mlp.down_proj.weight"]
    keys += ["model.norm.weight", "lm_head.weight"]
    d = tempfile.mkdtemp(prefix="cacti_ingest_")
    try:
        r = np.random.default_rng(0)
        hdr, off, blobs = {}, 0, []
        for key, (_, shp) in zip(keys, model.params):
            n = int(np.prod(shp))
            bits = (r.standard_normal(n, dtype=np.float32) * 0.02).view(np.uint32) >> 16     # bf16 bit patterns
            blobs.append(bits.astype(np.uint16))
            hdr[key] = {"dtype": "BF16", "shape": list(shp), "data_offsets": [off, off + 2 * n]}
            off += 2 * n
        pickled = args.ckpt_format == "pickle"
        if pickled:
            # pytorch_model.bin as torch.save writes it (the file PickleDir::open reads,
            # src/util/safepickle.rs:52-119); the bytes of each tensor are the same bf16 patterns
            import collections
            sd = collections.OrderedDict(
                (key, torch.from_numpy(b.view(np.int16)).view(torch.bfloat16).reshape(shp))
                for key, b, (_, shp) in zip(keys, blobs, model.params))
            torch.save(sd, os.path.join(d, "pytorch_model.bin"))
            del sd
        else:
            h = json.dumps(hdr).encode()
            with open(os.path.join(d, "model.safetensors"), "wb") as f:
                f.write(struct.pack("<Q", len(h)) + h)
                for b in blobs:
                    f.write(b.tobytes())
        nbytes = off

        def load():
            td = ingest.PickleDir(d) if pickled else ingest.TensorsDir(d)
            n = model.load_tensors_dir(td)
            ctx.sync()
            td.close()
            return n
        for _ in range(max(args.warmup, 1)):
            assert load() == len(keys)
        t0 = time.perf_counter()
        for _ in range(args.steps):
            load()
        dt = (time.perf_counter() - t0) / args.steps
        # the cells hold f16(bf16) of the file: lm_head against the oracle's cast
        want = o.raw_cast("bf16_f16", blobs[-1]).reshape(model.params[-1][1])
        got = model.param(len(keys) - 1)
        nan = np.isnan(want)
        assert np.array_equal(got[~nan].view(np.uint16), want[~nan].view(np.uint16))
        out = {"metric": "weight ingest: bf16 %s checkpoint -> f16 parameter cells on the device"
                         % ("torch (pickle)" if pickled else "safetensors"),
               "value": nbytes / dt / 1e9, "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": max(args.warmup, 1),
               "ms_per_step": dt * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
               "dtype": "u16", "data": "synthetic (N(0, 0.02) bf16 weights, file in the page cache)",
               "config": {"workload": "%d tensors, %.2f GB: embedding, %d layers, LM head of the 3B model"
                                      % (len(keys), nbytes / 1e9, cfg["L"])},
               "roofline": {"bound": "hbm", "achieved": 3 * nbytes / dt / 1e9, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                            "frac": 3 * nbytes / dt / 1e9 / PEAK_HBM_GBS, "traffic": None,
                            "note": "device bytes per checkpoint byte: staging write + cast read + cast write; the "
                                    "path is bound by the host copy and PCIe, not by HBM"}}
        if not args.no_cpu_baseline and not pickled:
            t0 = time.time()
            hd = o.read_safetensors_header(os.path.join(d, "model.safetensors"))
            mm = np.memmap(os.path.join(d, "model.safetensors"), dtype=np.uint8, mode="r")
            for k in keys:
                b, e = hd[k][2]
                o.raw_cast("bf16_f16", np.frombuffer(mm[b:e], dtype=np.uint16))
            t = time.time() - t0
            out["cpu_baseline"] = {"value": nbytes / t / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
                                   "sample": "oracle header read + bf16->f16 cast of the same file into host arrays (%.2f s)" % t}
        else:
            out["cpu_baseline"] = None
    finally:
        shutil.rmtree(d, ignore_errors=True)
    model.close()
    ctx.close()
    return out


def run_decode(args):
    """Single-stream greedy decoding with the key / value cache (examples/open_llama_3b_deploy.rs:195-206):
    a prompt of 1024 positions in one call, then one position per call, each feeding the previous
    call's arg max.  value = generated tokens per second over the timed single-position calls (each
    returns queued; one synchronisation at the end).  A position streams every weight matrix once
    (6.65 GB: all parameters but the embedding, of which one row is read) plus the cached keys and
    values of the positions before it."""
    import torch
    from cacti_amd.runtime import Ctx, Llama, LlamaCached
    cfg = dict(LLAMA_3B)
    if args.layers is not None:
        cfg["L"] = args.layers
    prompt = 1024
    steps = max(args.steps, 32)
    ctx = Ctx(0, 0, True)
    model = Llama(ctx, **cfg)
    synth_params(model)
    tok, _, _ = synth_inputs(cfg)
    k = LlamaCached(model, cfg["S"])
    k.set_tokens(tok[:prompt])
    k.apply(0, prompt)
    ctx.sync()
    t0 = time.perf_counter()
    k.reset_state()
    k.set_tokens(tok[:prompt])
    k.apply(0, prompt)
    ctx.sync()
    prefill = time.perf_counter() - t0
    pos = prompt
    for _ in range(max(args.warmup, 2)):
        k.apply(pos, pos + 1)
        pos += 1
    ctx.sync()
    torch.cuda.synchronize()
    first = pos
    t0 = time.perf_counter()
    for _ in range(steps):
        k.apply(pos, pos + 1)
        pos += 1
    ctx.sync()
    dt = (time.perf_counter() - t0) / steps
    toks = k.tokens()
    last = k.outputs(want_logit=False)["tok"]
    assert toks[pos] == last[0] and np.all(toks[pos + 1:] == 0) and np.array_equal(toks[:prompt], tok[:prompt])
    D, F, V, L = cfg["D"], cfg["F"], cfg["V"], cfg["L"]
    wbytes = 2 * (L * (4 * D * D + 3 * F * D + 2 * D) + D + V * D)
    ctx_mid = first + steps / 2.0
    kvbytes = 2 * 2 * L * ctx_mid * D
    out = {"metric": "greedy decoding tokens/sec with the key / value cache, 1 sequence", "value": 1.0 / dt,
           "unit": "tokens/s", "n_gpus": 1, "steps": steps, "warmup": max(args.warmup, 2), "ms_per_step": dt * 1e3,
           "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16",
           "data": "synthetic (seeded N(0,0.02) weights, uniform prompt ids)",
           "config": {"workload": "OpenLLaMA-3B shapes, %d layers, prompt %d positions then %d single positions "
                                  "(context %d .. %d), capacity %d" % (L, prompt, steps, first, pos, cfg["S"]),
                      "prefill_ms": prefill * 1e3, "prefill_tokens_per_s": prompt / prefill},
           "roofline": {"bound": "hbm", "achieved": (wbytes + kvbytes) / dt / 1e9, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                        "frac": (wbytes + kvbytes) / dt / 1e9 / PEAK_HBM_GBS, "traffic": None,
                        "note": "whole position: %.2f GB of weights + %.2f GB of cached keys and values over the "
                                "wall time of a call (about 15 launches per layer); per-kernel figures are in "
                                "profiles/" % (wbytes / 1e9, kvbytes / 1e9)}}
    k.close()
    model.close()
    ctx.close()
    if not args.no_cpu_baseline:
        from oracle import oracle as o
        from tests.llama_ref import make_inputs
        times = {}
        for Lc in (0, 2):
            ocfg, flat, otok, _, _ = make_inputs(dict(cfg, L=Lc), seed=0, norm_mean=1.0, grad_scale=1024.0)
            kc, vc = o.llama_cached_state(ocfg)
            it = np.zeros(ocfg.S, np.uint16)
            it[:8] = otok[:8]
            o.llama_cached_apply(ocfg, flat, kc, vc, it, 0, 8)
            t0 = time.time()
            for p in range(8, 12):
                o.llama_cached_apply(ocfg, flat, kc, vc, it, p, p + 1)
            times[Lc] = (time.time() - t0) / 4
        layer = max(times[2] - times[0], 1e-9) / 2
        full = times[0] + cfg["L"] * layer
        out["cpu_baseline"] = {"value": 1.0 / full, "unit": "tokens/s", "cores": o.num_threads(), "kind": "port",
                               "sample": "oracle cached pass, one position per call at full shapes: LM head alone (%.3f s) "
                                         "and with 2 layers (%.3f s per layer), extrapolated to %d layers"
                                         % (times[0], layer, cfg["L"])}
    else:
        out["cpu_baseline"] = None
    return out


def run_cycle(args):
    """The whole training cycle of the reference's example with one cycle per minibatch
    (examples/open_llama_3b_train.rs:223-531): fwd + loss + bwd, the numerical-health digests of every
    parameter and gradient, and the AdamW32 step on every parameter but the embedding; value = tokens
    per second over complete cycles, everything on the device (the reference runs the optimiser on the
    CPU)."""
    import torch
    from cacti_amd.runtime import Ctx, Llama
    cfg = dict(LLAMA_3B)
    if args.layers is not None:
        cfg["L"] = args.layers
    opt = dict(grad_scale=1024.0, lr=2.0e-5, wd=0.1, a1=0.1, a2=0.05, eps=1.0e-5)
    ctx = Ctx(0, 0, True)
    model = Llama(ctx, **cfg)
    synth_params(model)
    tok, lm_tok, scale = synth_inputs(cfg)
    model.adamw_init()

    def cycle(it):
        model.step(tok, lm_tok, scale, want_loss=False)
        gh, gn = model.digests(of_grads=True)
        ph, pn = model.digests(of_grads=False)
        model.adamw_step(it, skip_embed=True, **opt)
        return gh, gn, ph, pn
    it = 1
    for _ in range(max(args.warmup, 1)):
        cycle(it)
        it += 1
    ctx.sync()
    torch.cuda.synchronize()
    parts = {"step": 0.0, "digests": 0.0, "adamw": 0.0}
    t0 = time.perf_counter()
    for _ in range(args.steps):
        gh, gn, ph, pn = cycle(it)
        it += 1
    ctx.sync()
    dt = (time.perf_counter() - t0) / args.steps
    assert int(gn.sum()) == 0 and int(pn.sum()) == 0 and int(gh[:, 255].sum()) == 0, "non-finite values"
    # the three parts timed apart (each synchronised), for the breakdown only
    for _ in range(2):
        ta = time.perf_counter()
        model.step(tok, lm_tok, scale, want_loss=False)
        ctx.sync()
        tb = time.perf_counter()
        model.digests(of_grads=True)
        model.digests(of_grads=False)
        tc = time.perf_counter()
        model.adamw_step(it, skip_embed=True, **opt)
        it += 1
        ctx.sync()
        td = time.perf_counter()
        parts = {"step": (tb - ta) * 1e3, "digests": (tc - tb) * 1e3, "adamw": (td - tc) * 1e3}
    out = {"metric": "training-cycle tokens/sec: fwd+bwd, digests of parameters and gradients, AdamW32 step; 1 GPU",
           "value": cfg["S"] / dt, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": max(args.warmup, 1),
           "ms_per_step": dt * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16",
           "data": "synthetic (seeded N(0,0.02) weights, uniform token ids)",
           "config": {"workload": "OpenLLaMA-3B-shaped training cycle: %d layers, batch 1, seq %d, one cycle per "
                                  "minibatch, f32 master weights and moments on the device" % (cfg["L"], cfg["S"]),
                      "parts_ms": parts},
           "roofline": None, "cpu_baseline": None}
    model.close()
    ctx.close()
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=5)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--pool-gb", type=float, default=0.0,
                    help="cap of the device pool in GiB (0 = 90.01%% of the device); 16 exercises the host spill")
    ap.add_argument("--layers", type=int, default=None, help="override the layer count (debugging)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-capped", action="store_true", help="skip the second run on a pool capped at 16 GiB")
    ap.add_argument("--yardstick", action="store_true", help="gemm workload: also time the vendor library on each shape")
    ap.add_argument("--operands", choices=["randn", "zeros"], default="randn",
                    help="gemm workload: operand values (zeros: the rate without the power limit that real operands meet)")
    ap.add_argument("--sustain-probe", type=float, default=1.5, help="mfma-power workload: seconds per variant")
    ap.add_argument("--sustain", type=float, default=0.0, help="gemm workload: loop the largest product for this many seconds")
    ap.add_argument("--ckpt-format", choices=["safetensors", "pickle"], default="safetensors",
                    help="file format of the ingest workload's checkpoint")
    ap.add_argument("--workload", choices=["step", "adjoints", "gemm", "gemm-traffic", "gemm-step", "mfma-power", "attention", "digests", "adamw", "ingest",
                                           "decode", "cycle"], default="step")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        log("bench.py: this path runs on ONE GPU (the reference is single-device and the step "
            "has no collective); --gpus %d is not supported" % args.gpus)
        sys.exit(2)
    from cacti_amd import build
    build.ensure()                        # loads what is built; compiles only if nothing is
    if args.workload == "step":
        out = run_step(args)
    elif args.workload == "adjoints":
        out = run_adjoints(args)
    elif args.workload == "digests":
        out = run_digests(args)
    elif args.workload == "adamw":
        out = run_adamw(args)
    elif args.workload == "ingest":
        out = run_ingest(args)
    elif args.workload == "decode":
        out = run_decode(args)
    elif args.workload == "cycle":
        out = run_cycle(args)
    elif args.workload == "attention":
        out = run_attention(args)
    elif args.workload == "gemm-step":
        out = run_gemm_step(args)
    elif args.workload == "gemm-traffic":
        out = run_gemm_traffic(args)
    elif args.workload == "mfma-power":
        out = run_mfma_power(args)
    else:
        out = run_gemm(args)
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
