"""KV-cached forward pass (LlamaCached::apply, src/librarium/llama.rs:805-963; the row-causal mask,
src/librarium/llama.rs:1052-1112).

CPU: the oracle's cached pass is pinned against the oracle's own full forward pass, which other tests
pin: one call over the whole sequence reproduces its logits bit for bit (same thunks; the row-causal
mask with initial row 0 is the causal mask), and any split into chunks reproduces the one-call result
bit for bit (rows of a product do not depend on how many rows are computed with them), which fixes the
offsets of the cache rows, of the position tables and of the mask.  GPU: the HIP pass against the
oracle, chunk by chunk."""
import numpy as np
import pytest

from tests.util import assert_parity, rng


def _inputs(seed=4):
    from tests.test_gpu_llama import TINY, make_inputs
    return make_inputs(TINY, seed=seed, norm_mean=1.0, grad_scale=1024.0)


def test_oracle_cached_pass_equals_the_full_forward_pass(oracle):
    cfg, flat, tok, lm_tok, scale = _inputs()
    ref = oracle.llama_step(cfg, flat, tok, lm_tok, scale, want_grad=False)
    kc, vc = oracle.llama_cached_state(cfg)
    full = oracle.llama_cached_apply(cfg, flat, kc, vc, tok.copy(), 0, cfg.S, want_prob=True)
    assert np.array_equal(full["logit"].view(np.uint16), ref["logit"].view(np.uint16))
    assert np.array_equal(full["tok"], ref["amax"])
    assert np.allclose(full["prob"].sum(axis=1), 1.0, atol=1e-5)
    assert np.array_equal(full["prob"].argmax(axis=1), full["tok"])
    # the caches hold every position's rotated keys and plain values
    assert np.mean(kc != 0) > 0.99 and np.mean(vc != 0) > 0.99
    # chunks of any size, including single rows, give the same bits and the same caches
    kc2, vc2 = oracle.llama_cached_state(cfg)
    cuts = [0, 5, 6, 7, 40, cfg.S - 3, cfg.S]
    parts = []
    for a, b in zip(cuts[:-1], cuts[1:]):
        it = tok.copy()
        out = oracle.llama_cached_apply(cfg, flat, kc2, vc2, it, a, b)
        parts.append(out["logit"])
        if b < cfg.S:                                     # the generated token is added to the next input slot
            assert it[b] == (int(tok[b]) + int(out["tok"][-1])) % 65536
            assert np.array_equal(np.delete(it, b), np.delete(tok, b))
    assert np.array_equal(np.concatenate(parts).view(np.uint16), full["logit"].view(np.uint16))
    assert np.array_equal(kc, kc2) and np.array_equal(vc, vc2)
    # rows beyond `next` of a partly filled cache stay zero
    kc3, vc3 = oracle.llama_cached_state(cfg)
    oracle.llama_cached_apply(cfg, flat, kc3, vc3, tok.copy(), 0, 9)
    assert np.all(kc3[:, 9:] == 0) and np.all(vc3[:, 9:] == 0) and np.array_equal(kc3[:, :9], kc[:, :9])


def test_oracle_row_causal_mask(oracle):
    import ctypes as C
    T, H, Cc = 3, 2, 7
    x = np.arange(T * H * Cc, dtype=np.float32).reshape(T, H, Cc) + 1
    for row0 in (0, 2, 6, 100):
        y = np.empty_like(x)
        oracle.lib().th_row_causal_mask_f32(oracle.i64(T), oracle.i64(H), oracle.i64(Cc), oracle.i64(row0), oracle.P(x), oracle.P(y))
        for t in range(T):
            live = min(Cc, t + row0 + 1)
            assert np.array_equal(y[t, :, :live], x[t, :, :live]) and np.all(np.isneginf(y[t, :, live:]))


# ------------------------------------------------------------------------------------------ GPU
def _row_softmax_oracle(oracle, s16, row0):
    T, H, Cc = s16.shape
    s32 = s16.astype(np.float32)
    m = np.empty_like(s32)
    oracle.lib().th_row_causal_mask_f32(oracle.i64(T), oracle.i64(H), oracle.i64(Cc), oracle.i64(row0), oracle.P(s32), oracle.P(m))
    p = np.empty_like(s32)
    oracle.lib().th_softmax_f32(oracle.i64(T * H), oracle.i64(Cc), oracle.P(m), oracle.P(p))
    return oracle.cast_f32_f16(p)


@pytest.mark.gpu
@pytest.mark.parametrize("T,H,Cc,row0", [(1, 4, 8, 0), (1, 32, 2048, 2047), (1, 32, 1032, 1024), (5, 3, 520, 100),
                                         (64, 4, 64, 0), (3, 2, 16, 40)])
def test_row_causal_softmax_matches_the_oracle(oracle, T, H, Cc, row0):
    import torch
    from cacti_amd import ffi
    print("row causal softmax", T, H, Cc, row0, flush=True)
    r = rng(T + H + Cc + row0)
    s16 = (r.standard_normal((T, H, Cc)) * 3).astype(np.float16)
    want = _row_softmax_oracle(oracle, s16, row0)
    d = torch.from_numpy(s16.view(np.int16)).cuda()
    out = torch.full_like(d, 0x7e00)                       # NaN patterns: every column must be written
    ffi.call("cacti_hip_row_causal_softmax_fwd", T, H, Cc, Cc, row0, d.data_ptr(), out.data_ptr(), None)
    got = out.cpu().numpy().view(np.float16)
    assert_parity(got, want, "row causal softmax")
    live = np.arange(Cc)[None, :] <= (np.arange(T)[:, None] + row0)
    assert np.all(got[~np.broadcast_to(live[:, None, :], got.shape)] == 0)
    assert np.mean(got.view(np.uint16) == want.view(np.uint16)) > 0.99
    # in place
    ffi.call("cacti_hip_row_causal_softmax_fwd", T, H, Cc, Cc, row0, d.data_ptr(), d.data_ptr(), None)
    assert np.array_equal(d.cpu().numpy(), out.cpu().numpy())


@pytest.mark.gpu
@pytest.mark.parametrize("T,H,Dh,Cc,row0", [(1, 4, 64, 8, 0), (1, 32, 100, 2048, 2047), (1, 32, 100, 1031, 1030), (4, 3, 100, 300, 296),
                                            (2, 5, 36, 129, 50), (3, 2, 4, 700, 0), (1, 2, 100, 128, 127)])
def test_decoding_attention_matches_the_oracle_chain(oracle, T, H, Dh, Cc, row0):
    """scores -> mask -> softmax -> P V for one to four rows against the oracle's thunks over the
    whole cache; rows of the cache beyond the last position hold garbage that must not be read into
    the result; called twice on the same workspace."""
    import torch
    from cacti_amd import ffi
    print("attn decode", T, H, Dh, Cc, row0, flush=True)
    r = rng(T * 7 + H + Dh + Cc + row0)
    D = H * Dh
    q = (r.standard_normal((T, D))).astype(np.float16)
    kc = (r.standard_normal((Cc, D))).astype(np.float16)
    vc = (r.standard_normal((Cc, D))).astype(np.float16)
    alpha = 1.0 / np.sqrt(Dh)
    lib, i64, P = oracle.lib(), oracle.i64, oracle.P
    s16 = np.empty((T, H, Cc), np.float16)
    lib.th_block_matmul_f16(0, 1, i64(H), i64(T), i64(Cc), i64(Dh), oracle.f32(alpha), P(q), i64(D), i64(Dh), P(kc), i64(D), i64(Dh),
                            oracle.f32(0.0), P(s16), i64(H * Cc), i64(Cc))
    p16 = _row_softmax_oracle(oracle, s16, row0)
    want = np.empty((T, D), np.float16)
    lib.th_block_matmul_f16(0, 0, i64(H), i64(T), i64(Dh), i64(Cc), oracle.f32(1.0), P(p16), i64(H * Cc), i64(Cc), P(vc), i64(D), i64(Dh),
                            oracle.f32(0.0), P(want), i64(D), i64(Dh))
    live = min(Cc, T + row0)
    kc_d, vc_d = kc.copy(), vc.copy()
    kc_d[live:] = np.float16("nan")
    vc_d[live:] = np.float16("nan")
    dev = lambda a: torch.from_numpy(a.view(np.int16)).cuda()
    dq, dk, dv = dev(q), dev(kc_d), dev(vc_d)
    out = torch.zeros((T, D), dtype=torch.int16, device="cuda")
    nb = ffi.lib().cacti_hip_attn_decode_workspace(T, H, Dh, Cc)
    ws = torch.empty(nb, dtype=torch.uint8, device="cuda")
    for _ in range(2):
        ffi.call("cacti_hip_attn_decode_f16", T, H, Dh, Cc, row0, alpha, dq.data_ptr(), D, dk.data_ptr(), dv.data_ptr(), D, Dh,
                 out.data_ptr(), D, ws.data_ptr(), nb, None)
        got = out.cpu().numpy().view(np.float16)
        assert_parity(got, want, "attn decode")
        out.zero_()


@pytest.mark.gpu
@pytest.mark.parametrize("M,N,K,add,gate", [(1, 3200, 3200, False, False), (1, 8640, 3200, True, True), (2, 96, 256, True, False),
                                            (4, 250, 1024, False, True), (3, 32000, 3200, True, False), (1, 64, 8192, True, True),
                                            (1, 100, 136, False, False)])
def test_rows_norm_matmul_matches_the_separate_thunks(oracle, M, N, K, add, gate):
    """residual add -> RMSNorm -> product (-> SiLU gate with a second product) in one kernel against
    the oracle's thunks one after the other; the residual sum is stored bit-exactly."""
    import torch
    from cacti_amd import ffi
    print("rows norm matmul", M, N, K, add, gate, flush=True)
    r = rng(M + N + K + add + 2 * gate)
    x = r.standard_normal((M, K)).astype(np.float16)
    x2 = (r.standard_normal((M, K)) * 0.5).astype(np.float16) if add else None
    w = (1 + 0.1 * r.standard_normal(K)).astype(np.float16)
    B = (r.standard_normal((N, K)) * 0.05).astype(np.float16)
    B2 = (r.standard_normal((N, K)) * 0.05).astype(np.float16) if gate else None
    lib, i64, P, f32 = oracle.lib(), oracle.i64, oracle.P, oracle.f32
    rsum = x
    if add:
        rsum = np.empty_like(x)
        lib.th_add_f16(i64(M * K), P(x), P(x2), P(rsum))
    a = np.empty_like(x)
    ts, ss = np.empty((M, K), np.float32), np.empty(M, np.float32)
    lib.oracle_rmsnorm_fwd(i64(M), i64(K), P(rsum), P(w), f32(1e-6), P(a), P(ts), P(ss))
    want = oracle.matmul(0, 1, a, B)
    if gate:
        up = oracle.matmul(0, 1, a, B2)
        y, hh = np.empty_like(want), np.empty_like(want)
        lib.oracle_silu_gate_fwd(i64(M * N), P(want), P(up), P(y), P(hh))
        want = hh
    dev = lambda v: torch.from_numpy(v.view(np.int16)).cuda() if v is not None else None
    dx, dx2, dw, dB, dB2 = dev(x), dev(x2), dev(w), dev(B), dev(B2)
    out = torch.zeros((M, N), dtype=torch.int16, device="cuda")
    sout = torch.zeros((M, K), dtype=torch.int16, device="cuda") if add else None
    ptr = lambda v: v.data_ptr() if v is not None else None
    ffi.call("cacti_hip_rows_norm_matmul_f16", M, N, K, ptr(dx), ptr(dx2), ptr(dw), 1e-6, ptr(sout), ptr(dB), ptr(dB2),
             out.data_ptr(), None)
    got = out.cpu().numpy().view(np.float16)
    assert_parity(got, want, "rows norm matmul")
    assert np.mean(got.view(np.uint16) == want.view(np.uint16)) > 0.9        # the rest differ by one f16 ulp
    if add:
        assert np.array_equal(sout.cpu().numpy().view(np.uint16), rsum.view(np.uint16))
    # without the norm: the plain product of the (summed) rows
    if not add and not gate:
        ffi.call("cacti_hip_rows_norm_matmul_f16", M, N, K, ptr(dx), None, None, 0.0, None, ptr(dB), None, out.data_ptr(), None)
        assert_parity(out.cpu().numpy().view(np.float16), oracle.matmul(0, 1, x, B), "rows matmul")


@pytest.mark.gpu
@pytest.mark.parametrize("M,H,Dh,add", [(1, 32, 100, True), (1, 4, 64, False), (4, 6, 36, True), (2, 16, 128, False)])
def test_rows_qkv_rope_cache_matches_the_separate_thunks(oracle, M, H, Dh, add):
    """norm -> q, k, v products -> rotation -> cache accumulation in one launch against the oracle's
    thunks; the cache rows already hold values (the reference accumulates into them)."""
    import torch
    from cacti_amd import ffi
    print("rows qkv", M, H, Dh, add, flush=True)
    r = rng(M + H + Dh + add)
    D, pos0, cap = H * Dh, 5, 16
    x = r.standard_normal((M, D)).astype(np.float16)
    x2 = (r.standard_normal((M, D)) * 0.5).astype(np.float16) if add else None
    w = (1 + 0.1 * r.standard_normal(D)).astype(np.float16)
    Wq, Wk, Wv = ((r.standard_normal((D, D)) * 0.05).astype(np.float16) for _ in range(3))
    kc0, vc0 = ((r.standard_normal((M, D)) * 0.3).astype(np.float16) for _ in range(2))
    lib, i64, P, f32 = oracle.lib(), oracle.i64, oracle.P, oracle.f32
    cos16, sin16 = np.empty((cap, Dh), np.float16), np.empty((cap, Dh), np.float16)
    lib.oracle_rope_tables(i64(cap), i64(Dh), P(cos16), P(sin16))
    cr, sr = np.ascontiguousarray(cos16[pos0:pos0 + M]), np.ascontiguousarray(sin16[pos0:pos0 + M])
    rsum = x
    if add:
        rsum = np.empty_like(x)
        lib.th_add_f16(i64(M * D), P(x), P(x2), P(rsum))
    a = np.empty_like(x)
    ts, ss = np.empty((M, D), np.float32), np.empty(M, np.float32)
    lib.oracle_rmsnorm_fwd(i64(M), i64(D), P(rsum), P(w), f32(1e-6), P(a), P(ts), P(ss))
    q, kk, v = oracle.matmul(0, 1, a, Wq), oracle.matmul(0, 1, a, Wk), oracle.matmul(0, 1, a, Wv)
    qr, kr = np.empty_like(q), np.empty_like(kk)
    lib.oracle_rope_fwd(i64(M), i64(H), i64(Dh), P(q), P(cr), P(sr), P(qr))
    lib.oracle_rope_fwd(i64(M), i64(H), i64(Dh), P(kk), P(cr), P(sr), P(kr))
    want_k, want_v = np.empty_like(kc0), np.empty_like(vc0)
    lib.th_add_f16(i64(M * D), P(kc0), P(kr), P(want_k))
    lib.th_add_f16(i64(M * D), P(vc0), P(v), P(want_v))
    dev = lambda t_: torch.from_numpy(np.ascontiguousarray(t_).view(np.int16)).cuda() if t_ is not None else None
    ptr = lambda t_: t_.data_ptr() if t_ is not None else None
    dx, dx2, dw, dq, dk, dv, dc, ds, dkc, dvc = (dev(t_) for t_ in (x, x2, w, Wq, Wk, Wv, cr, sr, kc0, vc0))
    out = torch.zeros((M, D), dtype=torch.int16, device="cuda")
    sout = torch.zeros((M, D), dtype=torch.int16, device="cuda") if add else None
    ffi.call("cacti_hip_rows_qkv_rope_cache_f16", M, H, Dh, ptr(dx), ptr(dx2), ptr(dw), 1e-6, ptr(sout), ptr(dq), ptr(dk), ptr(dv),
             ptr(dc), ptr(ds), out.data_ptr(), ptr(dkc), ptr(dvc), None)
    h16 = lambda t_: t_.cpu().numpy().view(np.float16)
    assert_parity(h16(out), qr, "rotated queries")
    assert_parity(h16(dkc), want_k, "key cache rows")
    assert_parity(h16(dvc), want_v, "value cache rows")
    assert np.mean(h16(out).view(np.uint16) == qr.view(np.uint16)) > 0.95
    if add:
        assert np.array_equal(sout.cpu().numpy().view(np.uint16), rsum.view(np.uint16))


def _gpu_model(cfg, flat):
    from tests.test_gpu_llama import _model
    ctx, m = _model(cfg)
    m.put_params_flat(flat)
    return ctx, m


@pytest.mark.gpu
def test_cached_pass_matches_the_oracle_chunk_by_chunk(oracle):
    """Teacher-forced input: a prompt chunk, single tokens, a mid-sized chunk, the rest; logits,
    probabilities and arg-max tokens of every chunk against the oracle's cached pass."""
    from cacti_amd.runtime import LlamaCached
    cfg, flat, tok, lm_tok, scale = _inputs(seed=5)
    ctx, m = _gpu_model(cfg, flat)
    k = LlamaCached(m, cfg.S)
    kc, vc = oracle.llama_cached_state(cfg)
    cuts = [0, 13, 14, 15, 16, 48, 51, cfg.S]
    for a, b in zip(cuts[:-1], cuts[1:]):
        print("cached chunk", a, b, flush=True)
        k.set_tokens(tok)
        k.apply(a, b, want_prob=True)
        got = k.outputs()
        it = tok.copy()
        want = oracle.llama_cached_apply(cfg, flat, kc, vc, it, a, b, want_prob=True)
        assert_parity(got["logit"], want["logit"], "logit %d:%d" % (a, b))
        assert np.abs(got["prob"] - want["prob"]).max() < 2e-3 and np.allclose(got["prob"].sum(axis=1), 1, atol=1e-4)
        top2 = np.sort(want["logit"].astype(np.float32), axis=1)[:, -2:]
        clear = (top2[:, 1] - top2[:, 0]) > 0.02
        assert np.array_equal(got["tok"][clear], want["tok"][clear]) and clear.mean() > 0.5
        assert np.array_equal(got["tok"], got["logit"].astype(np.float32).argmax(axis=1))
        if b < cfg.S:                                     # the appended token
            toks = k.tokens()
            assert toks[b] == (int(tok[b]) + int(got["tok"][-1])) % 65536
            assert np.array_equal(np.delete(toks, b), np.delete(tok, b))
    k.close(); m.close(); ctx.close()


@pytest.mark.gpu
def test_cached_pass_in_one_call_matches_the_training_forward_pass(oracle):
    from cacti_amd.runtime import LlamaCached
    cfg, flat, tok, lm_tok, scale = _inputs(seed=6)
    ctx, m = _gpu_model(cfg, flat)
    k = LlamaCached(m, cfg.S)
    k.set_tokens(tok)
    k.apply(0, cfg.S)
    got = k.outputs()["logit"]
    # the cached pass runs the attention block as separate kernels: against the training pass staged
    # the same way nearly every logit is the same f16; the fused attention thunk rounds its softmax
    # differently in the last place, so there the bar is the parity tolerance alone
    for mode, same in (("thunks", 0.95), ("fused", 0.0)):
        m.set_attention(mode)
        m.step(tok, lm_tok, scale, want_grad=False)
        ref = ctx.cell_get(m.io_cells()["logit"], np.float16, (cfg.S, cfg.V))
        assert_parity(got, ref, "cached vs training forward, attention " + mode)
        assert np.mean(got.view(np.uint16) == ref.view(np.uint16)) > same
    k.close(); m.close(); ctx.close()


@pytest.mark.gpu
def test_greedy_generation_feeds_its_own_tokens(oracle):
    """The deploy loop (examples/open_llama_3b_deploy.rs:195-206): prompt, then one position per
    cycle; every cycle's input token is the previous cycle's arg max (asserted by the example), the
    cache is reset between two runs, and the run matches the oracle's while its arg max is clear."""
    from cacti_amd.runtime import LlamaCached
    cfg, flat, tok, lm_tok, scale = _inputs(seed=7)
    ctx, m = _gpu_model(cfg, flat)
    k = LlamaCached(m, cfg.S)
    P, n_new = 9, 12
    runs = []
    for _ in range(2):
        k.reset_state()
        k.set_tokens(tok[:P])
        k.apply(0, P)
        outs = [int(k.outputs(want_logit=False)["tok"][-1])]
        for i in range(1, n_new):
            k.apply(P + i - 1, P + i)
            outs.append(int(k.outputs(want_logit=False)["tok"][0]))
        toks = k.tokens()
        assert np.array_equal(toks[:P], tok[:P]) and list(toks[P:P + n_new]) == outs and np.all(toks[P + n_new:] == 0)
        runs.append(outs)
    assert runs[0] == runs[1]
    kc, vc = oracle.llama_cached_state(cfg)
    it = np.zeros(cfg.S, np.uint16)
    it[:P] = tok[:P]
    a, b = 0, P
    for i in range(n_new):
        want = oracle.llama_cached_apply(cfg, flat, kc, vc, it, a, b)
        top2 = np.sort(want["logit"][-1].astype(np.float32))[-2:]
        if top2[1] - top2[0] < 0.02 or int(want["tok"][-1]) != runs[0][i]:
            assert top2[1] - top2[0] < 0.02, (i, want["tok"][-1], runs[0][i])
            break
        a, b = b, b + 1
    assert i >= 2
    k.close(); m.close(); ctx.close()


@pytest.mark.gpu
def test_cached_pass_error_paths(oracle):
    from cacti_amd.ffi import CactiError
    from cacti_amd.runtime import LlamaCached
    cfg, flat, tok, lm_tok, scale = _inputs(seed=5)
    ctx, m = _gpu_model(cfg, flat)
    for bad_cap in (cfg.S + 8, 12, 0):
        with pytest.raises(CactiError) as e:
            LlamaCached(m, bad_cap)
        assert e.value.code == -1
    k = LlamaCached(m, 64)                                 # a capacity below the model's
    with pytest.raises(CactiError) as e:
        k.outputs()
    assert e.value.code == -5
    for a, b in ((0, 65), (-1, 3), (5, 5), (7, 3)):
        with pytest.raises(CactiError) as e:
            k.apply(a, b)
        assert e.value.code == -1, (a, b)
    with pytest.raises(CactiError) as e:
        k.set_tokens(np.zeros(65, np.uint16))
    assert e.value.code == -1
    bad = tok[:64].copy()
    bad[3] = cfg.V                                        # token id out of range: reported at the next sync
    k.set_tokens(bad)
    k.apply(0, 8)
    with pytest.raises(CactiError) as e:
        k.outputs()
    assert e.value.code == -3
    k.set_tokens(tok[:64])
    k.reset_state()
    k.apply(0, 64)                                         # next == capacity: nothing is appended
    out = k.outputs()
    assert np.array_equal(k.tokens(), tok[:64]) and np.isfinite(out["logit"].astype(np.float32)).all()
    k.close(); m.close(); ctx.close()


@pytest.mark.gpu
def test_full_size_decode_agrees_with_one_call_over_the_same_tokens():
    """3B shapes (hidden 3200, 32 heads x 100, ffn 8640, vocabulary 32000), 2 layers, capacity 2048,
    no oracle run: a 515-token sequence processed as prompt + three single-token cycles (the
    streaming product kernels and the attention over the cache at one row) gives the logits of one
    call over all 515 positions (the tiled kernels) up to summation order (the bar between two
    device paths is wider than against the oracle: both carry their own rounding)."""
    from cacti_amd.runtime import Ctx, Llama, LlamaCached
    cfg = dict(S=2048, D=3200, H=32, Dh=100, F=8640, V=32000, L=2)
    ctx = Ctx(0, 0, True)
    m = Llama(ctx, **cfg)
    r = np.random.default_rng(0)
    for i, (name, shp) in enumerate(m.params):
        w = r.standard_normal(shp, dtype=np.float32) * 0.02
        if name.endswith("norm"):
            w += 1.0
        m.put_param(i, w.astype(np.float16))
    tok = r.integers(0, cfg["V"], 515).astype(np.uint16)
    k = LlamaCached(m, 2048)
    k.set_tokens(tok)
    k.apply(0, 515)
    ref = k.outputs()["logit"]
    k.reset_state()
    k.set_tokens(tok)
    k.apply(0, 512)
    head = k.outputs()["logit"]
    rows = [head]
    for p in (512, 513, 514):
        print("decode position", p, flush=True)
        k.set_tokens(tok)
        k.apply(p, p + 1)
        rows.append(k.outputs()["logit"])
    got = np.concatenate(rows)
    assert np.isfinite(ref.astype(np.float32)).all()
    assert_parity(got[:512], ref[:512], "prefill rows")
    # two summation orders of the same fp32 products, each rounded to f16 after every thunk: the
    # distance between them is twice the distance of either from exact arithmetic
    assert_parity(got[512:], ref[512:], "decoded rows", l2=3e-3, mx=6e-2)
    k.close(); m.close(); ctx.close()


@pytest.mark.gpu
def test_handles_of_freed_caches_stay_dead(oracle):
    """The caches are cells that live across cycles; once the cached model is closed their handles must name
    dead cells for good, not the cells a later cycle happens to create."""
    import ctypes as C
    from cacti_amd import ffi
    from cacti_amd.runtime import LlamaCached
    cfg, flat, tok, lm_tok, scale = _inputs(seed=2)
    ctx, m = _gpu_model(cfg, flat)
    m.step(tok, lm_tok, scale, want_grad=False)

    def live(i):
        n = C.c_size_t()
        return ffi.lib().cacti_cell_bytes(ctx._c, i, C.byref(n)) == 0

    top0 = max(i for i in range(1, 4096) if live(i))
    k = LlamaCached(m, cfg.S)
    k.set_tokens(tok)
    k.apply(0, 4)
    k.outputs()
    caches = [i for i in range(top0 + 1, top0 + 4096) if live(i)]
    assert len(caches) >= 2 * cfg.L
    k.close()
    for _ in range(2):
        m.step(tok, lm_tok, scale)                    # reset + a new cycle's cells
        assert not any(live(i) for i in caches)
    m.close(); ctx.close()
