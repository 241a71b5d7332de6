"""Weight ingest: safetensors directory -> parameter cells (TensorsDir, src/util/safetensor.rs:45-160;
CellMatcher, src/util/cell.rs:47-112; Llama::match_pickle_dir, src/librarium/llama.rs:284-302;
resume_put, src/spine.rs:1714-1745; the bf16 raw casts, src/thunk/op.rs:665-803).

CPU: the oracle's casts against independent numpy derivations over every 16-bit pattern; the oracle's
matcher against hand-written expectations on Hugging Face LLaMA tensor names (including the quirks that
follow from scanning sorted keys); the product's host code (C ABI, no GPU call) against the oracle's
matcher on random cases and against files written by the `safetensors` package, an independent
implementation of the format.  GPU: the cast kernels bit for bit, and a tiny model loaded from F16,
BF16 and F32 files."""
import json
import os
import struct

import numpy as np
import pytest

from tests.util import rng


def hf_keys(num_layers, with_rotary=True):
    keys = ["model.embed_tokens.weight", "model.norm.weight", "lm_head.weight"]
    for i in range(num_layers):
        p = "model.layers.%d." % i
        keys += [p + "input_layernorm.weight", p + "post_attention_layernorm.weight", p + "self_attn.q_proj.weight",
                 p + "self_attn.k_proj.weight", p + "self_attn.v_proj.weight", p + "self_attn.o_proj.weight",
                 p + "mlp.gate_proj.weight", p + "mlp.up_proj.weight", p + "mlp.down_proj.weight"]
        if with_rotary:
            keys.append(p + "self_attn.rotary_emb.inv_freq")
    return keys


def hf_expected(num_layers):
    want = ["model.embed_tokens.weight"]
    for i in range(num_layers):
        p = "model.layers.%d." % i
        want += [p + "input_layernorm.weight", p + "self_attn.q_proj.weight", p + "self_attn.k_proj.weight",
                 p + "self_attn.v_proj.weight", p + "self_attn.o_proj.weight", p + "post_attention_layernorm.weight",
                 p + "mlp.gate_proj.weight", p + "mlp.up_proj.weight", p + "mlp.down_proj.weight"]
    return want + ["model.norm.weight", "lm_head.weight"]


# ------------------------------------------------------------------------------------------ oracle
def test_oracle_raw_casts_over_all_patterns(oracle):
    u = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    as32 = (u.astype(np.uint32) << 16).view(np.float32)
    got32 = oracle.raw_cast("bf16_f32", u)
    assert np.array_equal(got32.view(np.uint32), as32.view(np.uint32))
    with np.errstate(over="ignore"):
        want16 = as32.astype(np.float16)                    # numpy rounds to nearest even, overflow -> inf
    got16 = oracle.raw_cast("bf16_f16", u)
    fin = ~np.isnan(as32)
    assert np.array_equal(got16[fin].view(np.uint16), want16[fin].view(np.uint16))
    assert np.all(np.isnan(got16[~fin]))
    # bf16 -> f32 -> bf16 and f16 -> bf16 are truncations: exact on representable values, never away
    # from zero, less than one bf16 ulp (2^-7 relative) short
    assert np.array_equal(oracle.raw_cast("f32_bf16", as32), u)
    r = rng(5)
    x = (r.standard_normal(100000) * np.exp(r.uniform(-30, 30, 100000))).astype(np.float32)
    t = oracle.raw_cast("bf16_f32", oracle.raw_cast("f32_bf16", x))
    assert np.all(np.abs(t) <= np.abs(x)) and np.all(np.sign(t) == np.sign(x))
    assert np.all(np.abs(x) - np.abs(t) < np.abs(x) * 2.0 ** -7)
    h = u.view(np.float16)
    hb = oracle.raw_cast("f16_bf16", h)
    fin = np.isfinite(h)
    t = oracle.raw_cast("bf16_f32", hb)
    hf = h.astype(np.float32)
    assert np.all(np.abs(t[fin]) <= np.abs(hf[fin])) and np.all(np.abs(hf[fin]) - np.abs(t[fin]) <= np.abs(hf[fin]) * 2.0 ** -7)
    assert np.array_equal(np.isnan(t), np.isnan(hf)) and np.array_equal(np.isinf(t), np.isinf(hf))
    few_bits = fin & ((u & 0x7) == 0) & ((u & 0x7c00) != 0)       # normal f16 with 7 mantissa bits: exact
    assert np.array_equal(t[few_bits], hf[few_bits])


def test_oracle_matcher_on_hugging_face_names(oracle):
    for L in (1, 2, 12):
        got = oracle.cell_matcher_match(hf_keys(L), oracle.llama_rules(L))
        assert got == hf_expected(L), L
    # layer 1 never takes layer 10's or 11's tensors (an integer needs the whole token)
    got = oracle.cell_matcher_match(hf_keys(12), [(1, "attn", "q_proj"), (11, "mlp", "up"), (1, "mlp", "up")])
    assert got == ["model.layers.1.self_attn.q_proj.weight", "model.layers.11.mlp.up_proj.weight",
                   "model.layers.1.mlp.up_proj.weight"]
    # a string matches by containment, scanning sorted keys: with the layer norms still in the set,
    # "norm" takes the first of them, not model.norm.weight
    assert oracle.cell_matcher_match(hf_keys(2), [("norm",)]) == ["model.layers.0.input_layernorm.weight"]
    # ... which is what happens to the head norm when the file has more layers than the model
    got = oracle.cell_matcher_match(hf_keys(3), oracle.llama_rules(2))
    assert got[-2] == "model.layers.2.input_layernorm.weight" and got[-1] == "lm_head.weight"
    # a matched key leaves the set; a rule without a key gives None; pattern elements match in order
    assert oracle.cell_matcher_match(["a.b", "a.c"], [("a",), ("a",), ("a",)]) == ["a.b", "a.c", None]
    assert oracle.cell_matcher_match(["x.proj.attn.0"], [(0, "attn"), ("attn", 0)]) == [None, "x.proj.attn.0"]
    assert oracle.cell_matcher_match([], [("a",)]) == [None]


def test_oracle_header_reader_agrees_with_the_safetensors_package(oracle, tmp_path):
    from safetensors import safe_open
    from safetensors.numpy import save_file
    r = rng(2)
    tensors = {"b.weight": r.standard_normal((3, 5)).astype(np.float16), "a": r.standard_normal(7).astype(np.float32),
               "c.d.e": np.arange(6, dtype=np.int32).reshape(1, 2, 3)}
    p = str(tmp_path / "x.safetensors")
    save_file(tensors, p, metadata={"format": "pt"})
    hdr = oracle.read_safetensors_header(p)
    raw = open(p, "rb").read()
    with safe_open(p, framework="numpy") as f:
        assert sorted(hdr) == sorted(f.keys())
        for k in f.keys():
            dt, shape, (b, e) = hdr[k]
            want = f.get_tensor(k)
            assert shape == want.shape and dt == {"float16": "F16", "float32": "F32", "int32": "I32"}[str(want.dtype)]
            assert raw[b:e] == want.tobytes()


# ------------------------------------------------------------------------------------------ host code through the C ABI
@pytest.fixture(scope="module")
def ingest():
    from cacti_amd import ingest as m
    return m


def test_matcher_equals_the_oracle(oracle, ingest):
    for L in (1, 2, 12):
        assert ingest.cell_matcher_match(hf_keys(L), oracle.llama_rules(L)) == hf_expected(L)
    assert ingest.cell_matcher_match(hf_keys(3), oracle.llama_rules(2)) == oracle.cell_matcher_match(hf_keys(3), oracle.llama_rules(2))
    r = rng(8)
    words = ["attn", "mlp", "norm", "layer", "proj", "q", "k", "up", "0", "1", "10", "11", "2", "embed", "x"]
    for _ in range(300):
        keys = list({".".join(r.choice(words, size=r.integers(1, 5))) for _ in range(r.integers(0, 12))})
        rules = []
        for _ in range(r.integers(1, 8)):
            rules.append(tuple(int(w) if w.isdigit() and r.random() < 0.7 else str(w)
                               for w in r.choice(words, size=r.integers(1, 4))))
        assert ingest.cell_matcher_match(keys, rules) == oracle.cell_matcher_match(keys, rules), (keys, rules)


def _write_raw(path, header, data):
    h = json.dumps(header).encode()
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(h)) + h + data)


def test_tensors_dir_reads_what_the_safetensors_package_wrote(oracle, ingest, tmp_path):
    from safetensors.numpy import save_file
    r = rng(3)
    one = {"model.b": r.standard_normal((4, 6)).astype(np.float16), "model.a": r.standard_normal((2, 3, 5)).astype(np.float32),
           "z": np.arange(10, dtype=np.int64), "empty": np.zeros((0, 4), np.float16)}
    d1 = tmp_path / "single"
    d1.mkdir()
    save_file(one, str(d1 / "model.safetensors"), metadata={"format": "pt", "note": "{}[],\"\\"})
    for path in (d1, d1 / "model.safetensors"):
        td = ingest.TensorsDir(path)
        assert td.keys() == sorted(one, key=lambda k: k.encode())
        hdr = oracle.read_safetensors_header(str(d1 / "model.safetensors"))
        for k, v in one.items():
            dt, arr = td.get(k)
            assert dt == hdr[k][0] and arr.shape == v.shape and arr.tobytes() == v.tobytes()
        td.close()
    # shards: taken in sorted file order, names merged
    d2 = tmp_path / "shards"
    d2.mkdir()
    save_file({"w2": one["model.b"]}, str(d2 / "model-00002-of-00002.safetensors"))
    save_file({"w1": one["model.a"], "w0": one["z"]}, str(d2 / "model-00001-of-00002.safetensors"))
    td = ingest.TensorsDir(d2)
    assert td.keys() == ["w0", "w1", "w2"] and td.get("w2")[1].tobytes() == one["model.b"].tobytes()
    td.close()
    # bf16 comes back as bit patterns
    bits = r.integers(0, 65536, 12).astype(np.uint16)
    _write_raw(str(tmp_path / "bf.safetensors"), {"t": {"dtype": "BF16", "shape": [3, 4], "data_offsets": [0, 24]}}, bits.tobytes())
    td = ingest.TensorsDir(tmp_path / "bf.safetensors")
    dt, arr = td.get("t")
    assert dt == "BF16" and np.array_equal(arr.reshape(-1), bits)
    td.close()


def test_tensors_dir_errors(ingest, tmp_path):
    from cacti_amd.ffi import CactiError
    from safetensors.numpy import save_file

    def code(path):
        with pytest.raises(CactiError) as e:
            ingest.TensorsDir(path)
        return e.value.code

    assert code(tmp_path / "nothing") == -6
    (tmp_path / "emptydir").mkdir()
    assert code(tmp_path / "emptydir") == -6
    x = np.ones((2, 2), np.float16)
    d = tmp_path / "dup"
    d.mkdir()
    save_file({"same": x}, str(d / "model-00001-of-00002.safetensors"))
    save_file({"same": x}, str(d / "model-00002-of-00002.safetensors"))
    assert code(d) == -7                                                # TensorsDirErr::DuplicateName
    ok = {"t": {"dtype": "F16", "shape": [2, 2], "data_offsets": [0, 8]}}
    _write_raw(str(tmp_path / "short.safetensors"), ok, b"\0" * 7)       # data range beyond the file
    assert code(tmp_path / "short.safetensors") == -7
    _write_raw(str(tmp_path / "size.safetensors"), {"t": dict(ok["t"], shape=[3, 2])}, b"\0" * 8)   # range != type size
    assert code(tmp_path / "size.safetensors") == -7
    _write_raw(str(tmp_path / "dtype.safetensors"), {"t": dict(ok["t"], dtype="Q4")}, b"\0" * 8)
    assert code(tmp_path / "dtype.safetensors") == -7
    open(str(tmp_path / "tiny.safetensors"), "wb").write(b"abc")
    assert code(tmp_path / "tiny.safetensors") == -7
    open(str(tmp_path / "hlen.safetensors"), "wb").write(struct.pack("<Q", 1 << 40) + b"{}")
    assert code(tmp_path / "hlen.safetensors") == -7
    open(str(tmp_path / "json.safetensors"), "wb").write(struct.pack("<Q", 5) + b'{"t":')
    assert code(tmp_path / "json.safetensors") == -7
    _write_raw(str(tmp_path / "none.safetensors"), {}, b"")
    td = ingest.TensorsDir(tmp_path / "none.safetensors")
    assert td.keys() == []
    td.close()


# ------------------------------------------------------------------------------------------ GPU
@pytest.mark.gpu
@pytest.mark.parametrize("n", [0, 1, 3, 4, 5, 65536, 8192 * 3 + 2])
def test_raw_casts_match_the_oracle_bit_for_bit(oracle, n):
    import torch
    from cacti_amd import ops
    r = rng(40 + n % 7)
    print("raw casts", n, flush=True)
    u = np.arange(65536, dtype=np.uint32).astype(np.uint16) if n == 65536 else r.integers(0, 65536, n).astype(np.uint16)
    du = torch.from_numpy(u.view(np.int16)).cuda()
    g16 = ops.raw_cast_bf16_f16(du).cpu().numpy()
    w16 = oracle.raw_cast("bf16_f16", u)
    nan = np.isnan(w16)
    assert np.array_equal(np.isnan(g16), nan) and np.array_equal(g16[~nan].view(np.uint16), w16[~nan].view(np.uint16))
    assert np.array_equal(ops.raw_cast_bf16_f32(du).cpu().numpy().view(np.uint32), oracle.raw_cast("bf16_f32", u).view(np.uint32))
    x = (r.standard_normal(n) * np.exp(r.uniform(-40, 40, n))).astype(np.float32)
    x[::5] = (u[::5].astype(np.uint32) << 16).view(np.float32)            # includes inf / nan / subnormal patterns
    assert np.array_equal(ops.raw_cast_f32_bf16(torch.from_numpy(x).cuda()).cpu().numpy().view(np.uint16),
                          oracle.raw_cast("f32_bf16", x))
    h = u.view(np.float16)
    gb, wb = ops.raw_cast_f16_bf16(torch.from_numpy(h.view(np.int16)).cuda().view(torch.float16)).cpu().numpy().view(np.uint16), \
        oracle.raw_cast("f16_bf16", h)
    hn = np.isnan(h)
    assert np.array_equal(gb[~hn], wb[~hn])
    assert np.all((gb[hn] & 0x7f80) == 0x7f80) and np.all((gb[hn] & 0x7f) != 0)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["F16", "BF16", "F32"])
def test_model_loads_its_parameters_from_a_safetensors_directory(oracle, ingest, tmp_path, dtype):
    """Hugging Face names, two shards, extra tensors the rules ignore: every parameter holds the
    file's values (through the cast the reference would stage for that dtype), and a cycle on the
    loaded model gives the same loss, bit for bit, as one on parameters put directly."""
    from tests.test_gpu_llama import TINY, _model, make_inputs
    cfg, flat, tok, lm_tok, scale = make_inputs(TINY, seed=8, norm_mean=1.0, grad_scale=1024.0)
    want = oracle.split_params(cfg, flat)
    L = int(cfg.L)
    names = ["embed"] + ["l%d.%s" % (i, s) for i in range(L) for s in
                         ("pre_norm", "q", "k", "v", "o", "post_norm", "gate", "up", "down")] + ["head_norm", "lm_head"]
    r = rng(1)
    entries, blob = {}, b""
    expect = {}
    for name, key in zip(names, hf_expected(L)):
        w = want[name]
        if dtype == "F16":
            raw, expect[name] = w, w
        elif dtype == "F32":
            raw = (w.astype(np.float32) * (1 + r.standard_normal(w.shape).astype(np.float32) * 1e-4))
            expect[name] = oracle.cast_f32_f16(raw)
        else:
            raw = oracle.raw_cast("f32_bf16", w.astype(np.float32))
            expect[name] = oracle.raw_cast("bf16_f16", raw)
        entries[key] = (raw, dtype)
    entries["model.layers.0.self_attn.rotary_emb.inv_freq"] = (np.ones(4, np.float32), "F32")
    d = tmp_path / ("ckpt_" + dtype)
    d.mkdir()
    keys = sorted(entries)
    for shard, part in enumerate((keys[::2], keys[1::2])):
        hdr, data = {"__metadata__": {"format": "pt"}}, b""
        for k in part:
            raw, dt = entries[k]
            b = np.ascontiguousarray(raw).tobytes()
            hdr[k] = {"dtype": dt, "shape": list(raw.shape), "data_offsets": [len(data), len(data) + len(b)]}
            data += b
        _write_raw(str(d / ("model-%05d-of-00002.safetensors" % (shard + 1))), hdr, data)
    ctx, m = _model(cfg)
    td = ingest.TensorsDir(d)
    assert m.load_tensors_dir(td) == len(names)
    td.close()
    for i, (name, _) in enumerate(m.params):
        assert np.array_equal(m.param(i).view(np.uint16), expect[name].view(np.uint16)), name
    loss = m.step(tok, lm_tok, scale)
    ctx2, m2 = _model(cfg)
    for i, (name, _) in enumerate(m2.params):
        m2.put_param(i, expect[name])
    assert np.array_equal(m2.step(tok, lm_tok, scale).view(np.uint32), loss.view(np.uint32))
    m.close(); ctx.close(); m2.close(); ctx2.close()


@pytest.mark.gpu
def test_load_rejects_a_shape_mismatch_and_an_unsupported_dtype(oracle, ingest, tmp_path):
    from cacti_amd.ffi import CactiError
    from tests.test_gpu_llama import TINY, _model, make_inputs
    cfg, flat, *_ = make_inputs(TINY, seed=8)
    D = int(cfg.D)
    ctx, m = _model(cfg)
    _write_raw(str(tmp_path / "shape.safetensors"),
               {"model.norm.weight": {"dtype": "F16", "shape": [D + 1], "data_offsets": [0, 2 * (D + 1)]}}, b"\0" * (2 * (D + 1)))
    _write_raw(str(tmp_path / "dtype.safetensors"),
               {"model.norm.weight": {"dtype": "I16", "shape": [D], "data_offsets": [0, 2 * D]}}, b"\0" * (2 * D))
    for f, code in (("shape.safetensors", -1), ("dtype.safetensors", -2)):
        td = ingest.TensorsDir(tmp_path / f)
        with pytest.raises(CactiError) as e:
            m.load_tensors_dir(td)
        assert e.value.code == code, f
        td.close()
    # a file that matches only one parameter loads that one
    x = (rng(3).standard_normal(D)).astype(np.float16)
    _write_raw(str(tmp_path / "one.safetensors"),
               {"model.norm.weight": {"dtype": "F16", "shape": [D], "data_offsets": [0, 2 * D]}}, x.tobytes())
    td = ingest.TensorsDir(tmp_path / "one.safetensors")
    assert m.load_tensors_dir(td) == 1
    td.close()
    assert np.array_equal(m.param(len(m.params) - 2).view(np.uint16), x.view(np.uint16))
    m.close(); ctx.close()


def test_tensors_dir_entry_refuses_a_buffer_that_is_too_small(ingest, tmp_path):
    import ctypes as C
    from cacti_amd import ffi
    from cacti_amd.ffi import CactiError
    _write_raw(str(tmp_path / "one.safetensors"),
               {"a.rather.long.tensor.name": {"dtype": "F16", "shape": [2], "data_offsets": [0, 4]}}, b"\0" * 4)
    td = ingest.TensorsDir(tmp_path / "one.safetensors")
    name, dt = C.create_string_buffer(8), C.create_string_buffer(16)
    nd, shp, ptr, nb = C.c_int(), (C.c_int64 * 8)(), C.c_void_p(), C.c_uint64()
    with pytest.raises(CactiError) as e:
        ffi.call("cacti_tensors_dir_entry", td._d, 0, name, 8, dt, 16, C.byref(nd), shp, C.byref(ptr), C.byref(nb))
    assert e.value.code == -1
    ffi.call("cacti_tensors_dir_entry", td._d, 0, None, 0, dt, 16, C.byref(nd), shp, C.byref(ptr), C.byref(nb))
    assert dt.value == b"F16" and nd.value == 1 and nb.value == 4
    td.close()
