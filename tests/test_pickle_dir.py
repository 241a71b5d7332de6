"""PickleDir (src/util/safepickle.rs:52-195): the tensors of a torch checkpoint, found without running its pickle.

The reference's parser is a third-party crate outside its tree, so the checker here is torch itself: the
files are written by torch.save in this test and read back with torch.load(weights_only=True); names,
dtypes, shapes and every byte must agree with what the library maps.  The ZIP64 layout that archives above
4 GiB use is covered by rewriting a small archive with saturated 32-bit fields, built with struct below."""
import collections
import struct
import zipfile

import numpy as np
import pytest

from tests.test_ingest import hf_expected

torch = pytest.importorskip("torch")

_DT = {torch.float16: "F16", torch.bfloat16: "BF16", torch.float32: "F32", torch.float64: "F64", torch.int64: "I64",
       torch.int32: "I32", torch.int16: "I16", torch.int8: "I8", torch.uint8: "U8"}


@pytest.fixture(scope="module")
def ingest():
    from cacti_amd import ingest as m
    return m


def _bits(t):
    t = t.detach().contiguous()
    return t.view(torch.int16).numpy().view(np.uint16) if t.dtype == torch.bfloat16 else t.numpy()


def _check_against_torch(ingest, path, files, prefix=None):
    """every tensor torch.load finds in `files` is in the directory opened at `path`, byte for byte"""
    want = {}
    for f in files:
        for k, v in torch.load(str(f), weights_only=True).items():
            if isinstance(v, torch.Tensor):
                want[k] = v
    d = ingest.PickleDir(path, prefix)
    assert d.keys() == sorted(want)                      # the order CellMatcher scans
    for k, v in want.items():
        dt, arr = d.get(k)
        assert dt == _DT[v.dtype], k
        assert arr.shape == tuple(v.shape), k
        assert arr.tobytes() == _bits(v).tobytes(), k
        assert d.entries[k][2] % 64 == 0
    d.close()
    return want


def _state(seed=0):
    g = torch.Generator().manual_seed(seed)
    sd = collections.OrderedDict()
    sd["model.embed_tokens.weight"] = torch.randn(64, 24, generator=g).half()
    sd["model.layers.0.self_attn.q_proj.weight"] = torch.randn(24, 24, generator=g).bfloat16()
    sd["model.layers.0.mlp.up_proj.weight"] = torch.randn(3, 5, 7, generator=g).double()
    sd["model.norm.weight"] = torch.randn(24, generator=g)
    sd["ids"] = torch.arange(-5, 300)
    sd["i32"] = torch.arange(17, dtype=torch.int32)
    sd["i16"] = torch.arange(-9, 9, dtype=torch.int16)
    sd["i8"] = torch.arange(-128, 127, dtype=torch.int8)
    sd["u8"] = torch.arange(0, 255, dtype=torch.uint8)
    sd["wrapped"] = torch.nn.Parameter(torch.randn(4, 4, 4, generator=g).half())
    sd["scalar"] = torch.tensor(3.25)
    sd["empty"] = torch.zeros(0, 8, dtype=torch.float16)
    return sd


@pytest.mark.parametrize("protocol", [2, 4])
def test_pickle_dir_reads_what_torch_saved(ingest, tmp_path, protocol):
    """Protocol 2 is torch.save's default; protocol 4 adds FRAME, MEMOIZE, SHORT_BINUNICODE and STACK_GLOBAL
    (torch's own weights-only loader reads protocol 2 only, so the expected tensors come from that file)."""
    sd = _state()
    sd["not_a_tensor"] = {"step": 3, "names": ["a", "b"], "lr": 1e-3, "flag": True, "none": None, "big": 1 << 40, "neg": -7}
    ref = tmp_path / "ref.bin"
    torch.save(sd, str(ref))
    f = tmp_path / "pytorch_model.bin"
    torch.save(sd, str(f), pickle_protocol=protocol)
    want = _check_against_torch(ingest, tmp_path, [ref])
    assert len(want) == len(sd) - 1
    _check_against_torch(ingest, f, [ref])               # a file instead of a directory


def test_pickle_dir_reads_a_module_state_dict_and_shards(ingest, tmp_path):
    """Module.state_dict() carries a _metadata attribute (a BUILD on the OrderedDict); shards are taken in
    sorted order under a caller-chosen prefix."""
    torch.manual_seed(3)
    net = torch.nn.Sequential(torch.nn.Linear(8, 16), torch.nn.LayerNorm(16), torch.nn.Linear(16, 4)).half()
    d = tmp_path / "sharded"
    d.mkdir()
    sd = net.state_dict()
    keys = list(sd)
    a = collections.OrderedDict((k, sd[k]) for k in keys[:3])
    a._metadata = sd._metadata
    b = collections.OrderedDict((k, sd[k]) for k in keys[3:])
    torch.save(a, str(d / "ckpt-00001-of-00002.bin"))
    torch.save(b, str(d / "ckpt-00002-of-00002.bin"))
    torch.save({"decoy": torch.ones(3)}, str(d / "pytorch_model-00001-of-00001.bin"))
    want = _check_against_torch(ingest, d, [d / "ckpt-00001-of-00002.bin", d / "ckpt-00002-of-00002.bin"], prefix="ckpt")
    assert sorted(want) == sorted(keys)
    one = tmp_path / "one"
    one.mkdir()
    torch.save(sd, str(one / "pytorch_model.bin"))
    _check_against_torch(ingest, one, [one / "pytorch_model.bin"])


def test_pickle_dir_views_of_one_storage(ingest, tmp_path):
    """Tensors that share a storage are saved once with element offsets: a packed view that starts on a
    64-byte boundary and ends where the storage ends loads (storage_start, src/util/safepickle.rs:152-166)."""
    base = torch.arange(256, dtype=torch.float16)
    f = tmp_path / "views.bin"
    torch.save({"whole": base, "tail": base[64:].view(6, 32)}, str(f))
    d = ingest.PickleDir(f)
    dt, arr = d.get("tail")
    assert dt == "F16" and np.array_equal(arr, base[64:].view(6, 32).numpy())
    assert d.entries["tail"][2] - d.entries["whole"][2] == 128
    d.close()


def _zip64_rewrite(src, dst):
    """The records of `src` re-emitted as a ZIP64 archive: every 32-bit size and offset in the central
    directory saturated and carried in the ZIP64 extra field, a ZIP64 end record and its locator before
    the classic end record.  Record data keeps its 64-byte alignment."""
    out, central = bytearray(), []
    with zipfile.ZipFile(src) as z:
        for info in z.infolist():
            data, name = z.read(info.filename), info.filename.encode()
            pad = (-(len(out) + 30 + len(name) + 4)) % 64          # an extra field of id 0xCAFE pads the data start
            extra = struct.pack("<HH", 0xCAFE, pad) + b"\0" * pad
            lho = len(out)
            out += struct.pack("<IHHHHHIIIHH", 0x04034b50, 45, 0, 0, 0, 0x21, info.CRC, len(data), len(data), len(name), len(extra))
            out += name + extra
            assert len(out) % 64 == 0
            out += data
            z64 = struct.pack("<HHQQQ", 1, 24, len(data), len(data), lho)
            central.append(struct.pack("<IHHHHHHIIIHHHHHII", 0x02014b50, 45, 45, 0, 0, 0, 0x21, info.CRC, 0xffffffff, 0xffffffff,
                                       len(name), len(z64), 0, 0, 0, 0, 0xffffffff) + name + z64)
    cd_off = len(out)
    for c in central:
        out += c
    cd_size = len(out) - cd_off
    z64_eocd = len(out)
    out += struct.pack("<IQHHIIQQQQ", 0x06064b50, 44, 45, 45, 0, 0, len(central), len(central), cd_size, cd_off)
    out += struct.pack("<IIQI", 0x07064b50, 0, z64_eocd, 1)
    out += struct.pack("<IHHHHIIH", 0x06054b50, 0, 0, 0xffff, 0xffff, 0xffffffff, 0xffffffff, 0)
    open(dst, "wb").write(bytes(out))


def test_pickle_dir_zip64_archive(ingest, tmp_path):
    f = tmp_path / "small.bin"
    torch.save(_state(5), str(f))
    g = tmp_path / "zip64.bin"
    _zip64_rewrite(str(f), str(g))
    assert set(zipfile.ZipFile(str(g)).namelist()) == set(zipfile.ZipFile(str(f)).namelist())   # a well-formed archive
    a, b = ingest.PickleDir(f), ingest.PickleDir(g)
    assert a.keys() == b.keys() and len(a.keys()) == len(_state(5))
    for k in a.keys():
        (dta, xa), (dtb, xb) = a.get(k), b.get(k)
        assert dta == dtb and xa.shape == xb.shape and xa.tobytes() == xb.tobytes(), k
    a.close(); b.close()


def test_pickle_dir_errors(ingest, tmp_path):
    from cacti_amd.ffi import CactiError

    def code(path, prefix=None):
        with pytest.raises(CactiError) as e:
            ingest.PickleDir(path, prefix)
        return e.value.code

    assert code(tmp_path / "nothing") == -6
    (tmp_path / "emptydir").mkdir()
    assert code(tmp_path / "emptydir") == -6
    x = torch.arange(64, dtype=torch.float16).view(8, 8)
    torch.save({"t": x.t()}, str(tmp_path / "strided.bin"))                     # non-packed strides: refused as in the reference
    assert code(tmp_path / "strided.bin") == -2
    torch.save({"t": x.view(-1)[3:]}, str(tmp_path / "unaligned.bin"))           # first byte 6 bytes into the storage
    assert code(tmp_path / "unaligned.bin") == -7
    torch.save({"t": torch.zeros(4, dtype=torch.complex64)}, str(tmp_path / "complex.bin"))
    assert code(tmp_path / "complex.bin") == -2                                  # storage type outside the accepted set
    torch.save({"t": x}, str(tmp_path / "legacy.bin"), _use_new_zipfile_serialization=False)
    assert code(tmp_path / "legacy.bin") == -7
    d = tmp_path / "dup"
    d.mkdir()
    torch.save({"same": x}, str(d / "pytorch_model-00001-of-00002.bin"))
    torch.save({"same": x}, str(d / "pytorch_model-00002-of-00002.bin"))
    assert code(d) == -7                                                         # PickleDirErr::DuplicateName
    torch.save([x, x], str(tmp_path / "list.bin"))                               # the pickled value is no dictionary
    assert code(tmp_path / "list.bin") == -7
    open(str(tmp_path / "tiny.bin"), "wb").write(b"PK")
    assert code(tmp_path / "tiny.bin") == -7
    good = tmp_path / "good.bin"
    torch.save({"t": x}, str(good))
    raw = open(str(good), "rb").read()
    open(str(tmp_path / "cut.bin"), "wb").write(raw[:len(raw) // 2])             # the end record is gone
    assert code(tmp_path / "cut.bin") == -7
    # a pickle with an opcode the scanner does not read (protocol-0 INT) inside a well-formed archive
    with zipfile.ZipFile(str(tmp_path / "opcode.bin"), "w") as z:
        z.writestr("archive/data.pkl", b"\x80\x02}q\x00X\x01\x00\x00\x00aI12\ns.")
    assert code(tmp_path / "opcode.bin") == -7
    with zipfile.ZipFile(str(tmp_path / "short.bin"), "w") as z:                 # the pickle ends inside an opcode
        z.writestr("archive/data.pkl", b"\x80\x02}q\x00X\x09\x00\x00\x00a")
    assert code(tmp_path / "short.bin") == -7
    with zipfile.ZipFile(str(tmp_path / "deep.bin"), "w") as z:                  # 100000 nested one-tuples
        z.writestr("archive/data.pkl", b"\x80\x02N" + b"\x85" * 100000 + b".")
    assert code(tmp_path / "deep.bin") == -7
    with zipfile.ZipFile(str(tmp_path / "nopkl.bin"), "w") as z:
        z.writestr("archive/version", b"3\n")
    assert code(tmp_path / "nopkl.bin") == -7
    # a storage record shorter than the pickle says
    with zipfile.ZipFile(str(good)) as z, zipfile.ZipFile(str(tmp_path / "shortrec.bin"), "w") as w:
        for info in z.infolist():
            data = z.read(info.filename)
            w.writestr(info.filename, data[:-2] if "/data/" in info.filename else data)
    assert code(tmp_path / "shortrec.bin") == -7
    with zipfile.ZipFile(str(good)) as z, zipfile.ZipFile(str(tmp_path / "norec.bin"), "w") as w:
        for info in z.infolist():
            if "/data/" not in info.filename:
                w.writestr(info.filename, z.read(info.filename))
    assert code(tmp_path / "norec.bin") == -7


def _crafted(path, tensors, byteorder=None):
    """A torch-style archive written by hand, so that the numbers in its pickle can lie: tensors maps a name
    to (record bytes, storage numel, storage offset, shape, stride[, storage class]).  Records start 64-byte
    aligned."""
    import io
    import pickle

    class Storage:
        def __init__(self, key, numel, cls):
            self.key, self.numel, self.cls = key, numel, cls

    class Tensor:
        def __init__(self, st, off, shape, stride):
            self.a = (st, off, tuple(shape), tuple(stride), False, collections.OrderedDict())

        def __reduce__(self):
            return (torch._utils._rebuild_tensor_v2, self.a)

    class Pk(pickle.Pickler):
        def persistent_id(self, obj):
            return ("storage", obj.cls, obj.key, "cpu", obj.numel) if isinstance(obj, Storage) else None

    sd = collections.OrderedDict()
    for i, (name, (data, numel, off, shape, stride, *cls)) in enumerate(tensors.items()):
        sd[name] = Tensor(Storage(str(i), numel, cls[0] if cls else torch.HalfStorage), off, shape, stride)
    buf = io.BytesIO()
    Pk(buf, protocol=2).dump(sd)
    with zipfile.ZipFile(str(path), "w") as z:
        z.writestr("archive/data.pkl", buf.getvalue())
        if byteorder is not None:
            z.writestr("archive/byteorder", byteorder[0], compress_type=byteorder[1])
        for i, (data, *_) in enumerate(tensors.values()):
            info = zipfile.ZipInfo("archive/data/%d" % i)
            pos = z.fp.tell() + 30 + len(info.filename)
            pad = (-(pos + 4)) % 64
            info.extra = struct.pack("<HH", 0x4346, pad) + b"\0" * pad          # an unknown extra field as padding
            z.writestr(info, data)


def test_pickle_dir_refuses_numbers_that_wrap_or_point_outside(ingest, tmp_path):
    """The element counts of a checkpoint are 64-bit numbers the file's author chose: products that wrap and
    ranges outside the record must be refused, not turned into a mapping of other memory."""
    from cacti_amd.ffi import CactiError

    def code(path):
        with pytest.raises(CactiError) as e:
            ingest.PickleDir(path)
        return e.value.code

    x = np.arange(64, dtype=np.float16)
    ok = tmp_path / "honest.bin"
    _crafted(ok, {"t": (x.tobytes(), 64, 32, (4, 8), (8, 1))}, byteorder=(b"little", zipfile.ZIP_STORED))
    d = ingest.PickleDir(ok)                                         # the hand-written archive itself is read
    dt, arr = d.get("t")
    assert dt == "F16" and arr.tobytes() == x[32:].tobytes()
    d.close()
    cases = {
        "negative_numel": (x.tobytes(), -1, 0, (64,), (1,)),
        "numel_wraps": (b"", 1 << 61, 1 << 60, (0,), (1,), torch.DoubleStorage),   # 2^61 * 8 bytes == 0 == the record's size, mod 2^64
        "numel_short": (x.tobytes(), 65, 0, (65,), (1,)),
        "shape_wraps": (x.tobytes(), 64, 0, (1 << 32, 1 << 32), (1 << 32, 1)),
        "offset_past_end": (x.tobytes(), 64, 65, (0,), (1,)),
        "negative_offset": (x.tobytes(), 64, -64, (64,), (1,)),
        "too_long": (x.tobytes(), 64, 32, (33,), (1,)),
    }
    for name, t in cases.items():
        _crafted(tmp_path / (name + ".bin"), {"t": t})
        assert code(tmp_path / (name + ".bin")) == -7, name
    _crafted(tmp_path / "bo_deflated.bin", {"t": (x.tobytes(), 64, 0, (64,), (1,))}, byteorder=(b"little" * 40, zipfile.ZIP_DEFLATED))
    assert code(tmp_path / "bo_deflated.bin") == -7
    _crafted(tmp_path / "bo_big.bin", {"t": (x.tobytes(), 64, 0, (64,), (1,))}, byteorder=(b"big", zipfile.ZIP_STORED))
    assert code(tmp_path / "bo_big.bin") == -2
    # 42 bytes that claim to be a ZIP64 archive: the 64-bit end record cannot lie inside the file
    loc = struct.pack("<IIQI", 0x07064b50, 0, 0x10000000, 1)
    eocd = struct.pack("<IHHHHIIH", 0x06054b50, 0xffff, 0xffff, 0xffff, 0xffff, 0xffffffff, 0xffffffff, 0)
    open(str(tmp_path / "zip64_stub.bin"), "wb").write(loc + eocd)
    assert code(tmp_path / "zip64_stub.bin") == -7


def test_pickle_dir_survives_hostile_object_graphs(ingest, tmp_path):
    """Pickles whose values form cycles or chains of any depth: built through the memo, so that no single
    opcode nests deeply.  The library refuses or reads them; it neither recurses per level nor leaks."""
    from cacti_amd.ffi import CactiError

    def open_code(name, pkl):
        with zipfile.ZipFile(str(tmp_path / name), "w") as z:
            z.writestr("archive/data.pkl", pkl)
        try:
            ingest.PickleDir(tmp_path / name).close()
            return 0
        except CactiError as e:
            return e.code

    # a chain grown from its inner end: every new list is appended to the one before it, 300000 levels
    step = b"]" + b"r\x00\x00\x00\x00" + b"a" + b"0" + b"j\x00\x00\x00\x00"
    assert open_code("chain.bin", b"\x80\x02]" + b"r\x01\x00\x00\x00" + step * 300000 + b".") == -7
    # the same chain below a dictionary, which is what a checkpoint's top value must be: read, and empty
    grow = b"}q\x01" + b"X\x01\x00\x00\x00k" + b"]q\x00" + b"s" + b"h\x00" + step * 300000 + b"0h\x01."
    assert open_code("chain_in_dict.bin", b"\x80\x02" + grow) == 0
    assert open_code("self_list.bin", b"\x80\x02]q\x00h\x00a.") == -7                       # a list that holds itself
    assert open_code("self_dict.bin", b"\x80\x02}q\x00X\x01\x00\x00\x00kh\x00s.") == 0      # a dictionary that does
    two = b"\x80\x02]q\x00]q\x01h\x00a0h\x00h\x01a."                                        # two lists that hold each other
    assert open_code("cycle2.bin", two) == -7
    assert open_code("many.bin", b"\x80\x02" + b"]" * 5000000 + b".") == -7                  # more values than any checkpoint needs
    assert open_code("wide.bin", b"\x80\x02](" + b"N" + b"2" * 5000000 + b"e.") == -7         # ... or references to one


# ------------------------------------------------------------------------------------------ GPU
@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["F16", "BF16"])
def test_model_loads_its_parameters_from_a_torch_checkpoint(oracle, ingest, tmp_path, dtype):
    """pytorch_model.bin with Hugging Face names, as the training example opens it
    (examples/open_llama_3b_train.rs:88-132): every parameter cell holds the file's values, BF16 through
    the raw cast the reference stages."""
    from tests.test_gpu_llama import TINY, _model, make_inputs
    cfg, flat, tok, lm_tok, scale = make_inputs(TINY, seed=9, norm_mean=1.0, grad_scale=1024.0)
    want = oracle.split_params(cfg, flat)
    L = int(cfg.L)
    names = ["embed"] + ["l%d.%s" % (i, s) for i in range(L) for s in
                         ("pre_norm", "q", "k", "v", "o", "post_norm", "gate", "up", "down")] + ["head_norm", "lm_head"]
    sd, expect = collections.OrderedDict(), {}
    for name, key in zip(names, hf_expected(L)):
        w = torch.from_numpy(want[name].copy())
        if dtype == "F16":
            sd[key], expect[name] = w, want[name]
        else:
            sd[key] = w.bfloat16()
            expect[name] = oracle.raw_cast("bf16_f16", _bits(sd[key]))
    sd["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.ones(4)
    torch.save(sd, str(tmp_path / "pytorch_model.bin"))
    ctx, m = _model(cfg)
    pd = ingest.PickleDir(tmp_path)
    assert m.load_tensors_dir(pd) == len(names)
    pd.close()
    for i, (name, _) in enumerate(m.params):
        assert np.array_equal(m.param(i).view(np.uint16), expect[name].view(np.uint16)), name
    m.close(); ctx.close()
