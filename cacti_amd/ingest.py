"""Host side of weight ingest: TensorsDir (src/util/safetensor.rs:45-160), PickleDir
(src/util/safepickle.rs:52-195) and CellMatcher (src/util/cell.rs:47-112) through the C ABI of
include/cacti_hip_runtime.h."""
import ctypes as C

import numpy as np

from . import ffi

_NP = {"F16": np.float16, "F32": np.float32, "F64": np.float64, "BF16": np.uint16, "U16": np.uint16,
       "I16": np.int16, "I32": np.int32, "U32": np.uint32, "I64": np.int64, "U64": np.uint64, "I8": np.int8,
       "U8": np.uint8, "BOOL": np.uint8}


class TensorsDir:
    """TensorsDir::open + get: names in the order CellMatcher scans them, memory-mapped tensors."""

    def __init__(self, path):
        self._d = C.c_void_p()
        ffi.call("cacti_tensors_dir_open", str(path).encode(), C.byref(self._d))
        self._read_entries()

    def _read_entries(self):
        self.entries = {}             # name -> (dtype string, shape, address, bytes)
        name, dt = C.create_string_buffer(4096), C.create_string_buffer(16)
        for i in range(ffi.lib().cacti_tensors_dir_count(self._d)):
            nd, shp, ptr, nb = C.c_int(), (C.c_int64 * 8)(), C.c_void_p(), C.c_uint64()
            ffi.call("cacti_tensors_dir_entry", self._d, i, name, 4096, dt, 16, C.byref(nd), shp, C.byref(ptr),
                     C.byref(nb))
            self.entries[name.value.decode("utf-8", "surrogateescape")] = (dt.value.decode(), tuple(shp[k] for k in range(nd.value)),
                                                 ptr.value, nb.value)

    def keys(self):
        return list(self.entries)

    def get(self, key):
        """(dtype string, array copied out of the mapping); bf16 comes back as uint16 bit patterns."""
        dt, shape, addr, nb = self.entries[key]
        buf = (C.c_char * nb).from_address(addr) if nb else b""
        return dt, np.frombuffer(buf, dtype=_NP[dt]).reshape(shape).copy()

    def close(self):
        if self._d:
            ffi.lib().cacti_tensors_dir_close(self._d)
            self._d = None


class PickleDir(TensorsDir):
    """PickleDir::open / open_with_prefix + get: the tensors of pytorch_model.bin (or its shards), found
    by scanning the pickle without executing it; same table, same accessors as TensorsDir."""

    def __init__(self, path, prefix=None):
        self._d = C.c_void_p()
        ffi.call("cacti_pickle_dir_open", str(path).encode(), prefix.encode() if prefix else None, C.byref(self._d))
        self._read_entries()


def _rule(pat):
    pat = pat if isinstance(pat, tuple) else (pat,)
    return "/".join("#%d" % p if isinstance(p, int) else p for p in pat).encode()


def cell_matcher_match(keys, rules):
    """CellMatcher::match_: per rule (tuple of int / str patterns) the matched key or None."""
    nk, nr = len(keys), len(rules)
    ka = (C.c_char_p * max(nk, 1))(*[k.encode() for k in keys])
    ra = (C.c_char_p * max(nr, 1))(*[_rule(r) for r in rules])
    out = (C.c_int * max(nr, 1))()
    ffi.call("cacti_cell_matcher_match", C.cast(ka, C.c_void_p), nk, C.cast(ra, C.c_void_p), nr,
             C.cast(out, C.c_void_p))
    return [keys[out[r]] if out[r] >= 0 else None for r in range(nr)]
