"""The device pool's placement policy over a plain offset range (host only, no GPU):
256-byte granules, first fit over coalesced free regions, bump cursor, retraction.
Mirrors NvGpuMemPool's front allocator, src/pctx/nvgpu.rs:30, 1633-1655."""
import random

import pytest

from cacti_amd.runtime import MemPool


def test_alignment_bump_and_exhaustion():
    p = MemPool(4096)
    a = p.alloc(1)
    b = p.alloc(257)
    assert (a, b) == (0, 256)                       # 1 -> 256, 257 -> 512
    assert p.stats()["used"] == 768 and p.stats()["front"] == 768
    assert p.alloc(4096 - 768 + 1) is None          # does not fit: nothing changes
    assert p.stats()["used"] == 768
    c = p.alloc(4096 - 768)
    assert c == 768 and p.stats()["largest_free"] == 0
    assert p.alloc(1) is None


def test_first_fit_reuses_lowest_hole_and_splits():
    p = MemPool(1 << 20)
    offs = [p.alloc(1024) for _ in range(6)]
    p.free(offs[1])
    p.free(offs[3])
    assert p.alloc(2048) == 6 * 1024                # neither hole fits: bump
    assert p.alloc(512) == offs[1]                  # lowest hole, split
    assert p.alloc(512) == offs[1] + 512
    assert p.alloc(1024) == offs[3]


def test_coalescing_and_cursor_retraction():
    p = MemPool(1 << 20)
    a, b, c, d = (p.alloc(4096) for _ in range(4))
    p.free(b)
    p.free(c)                                       # b+c merge into one 8 KiB hole
    assert p.alloc(8192) == b
    p.free(b)
    p.free(d)                                       # hole now touches the cursor: retract
    assert p.stats()["front"] == 4096
    p.free(a)
    s = p.stats()
    assert s["front"] == 0 and s["used"] == 0 and s["largest_free"] == s["cap"]
    assert s["peak"] == 4 * 4096


def test_double_free_is_an_error():
    from cacti_amd.ffi import CactiError
    p = MemPool(4096)
    a = p.alloc(10)
    p.free(a)
    with pytest.raises(CactiError):
        p.free(a)


def test_random_workload_never_overlaps_and_accounts():
    rnd = random.Random(0)
    cap = 1 << 22
    p = MemPool(cap)
    live = {}
    for _ in range(4000):
        if live and rnd.random() < 0.45:
            off = rnd.choice(list(live))
            p.free(off)
            del live[off]
        else:
            n = rnd.choice([1, 100, 256, 4096, 70000, 300000])
            off = p.alloc(n)
            if off is None:
                assert p.stats()["largest_free"] < (n + 255) // 256 * 256
                continue
            size = (n + 255) // 256 * 256
            assert off % 256 == 0 and off + size <= cap
            for o, s in live.items():
                assert off + size <= o or o + s <= off, "overlap"
            live[off] = size
        assert p.stats()["used"] == sum(live.values())
    for off in list(live):
        p.free(off)
    assert p.stats()["front"] == 0


def test_high_end_mirrors_the_low_end():
    p = MemPool(1 << 20)
    a = p.alloc(1000, high=True)
    b = p.alloc(256, high=True)
    assert (a, b) == ((1 << 20) - 1024, (1 << 20) - 1280)
    lo = p.alloc(512)
    assert lo == 0 and p.stats()["front"] == 512
    assert p.stats()["largest_free"] == (1 << 20) - 1280 - 512
    p.free(a)                                          # a hole above the back cursor
    assert p.alloc(512, high=True) == (1 << 20) - 512  # its high end
    assert p.alloc(1024, high=True) == (1 << 20) - 1280 - 1024   # does not fit the rest: cursor
    p.free(b)
    assert p.alloc(256, high=True) == (1 << 20) - 768  # b's region merged with the rest of a's: its high end
    for off in (lo,):
        p.free(off)
    assert p.stats()["front"] == 0


def test_each_end_falls_back_to_the_others_holes():
    p = MemPool(4096)
    hi = [p.alloc(1024, high=True) for _ in range(3)]     # 3072..4095, 2048.., 1024..
    lo = p.alloc(1024)
    assert lo == 0 and p.alloc(256) is None and p.alloc(256, high=True) is None
    p.free(hi[1])                                         # a hole in the high part
    assert p.alloc(512) == hi[1]                          # low request: its low end
    p.free(lo)                                            # cursor retracts: room between the cursors
    assert p.alloc(1024, high=True) == 0                  # between the cursors
    assert p.alloc(512, high=True) == hi[1] + 512
    assert p.stats()["used"] == 4096 and p.alloc(1) is None


def test_random_two_ended_traffic_never_overlaps():
    r = random.Random(11)
    cap = 1 << 20
    p = MemPool(cap)
    live = {}
    for _ in range(4000):
        if live and (r.random() < 0.45 or len(live) > 60):
            off = r.choice(list(live))
            p.free(off)
            del live[off]
        else:
            n = r.choice((256, 512, 3 * 256, 4096, 20 * 1024, 55 * 1024))
            off = p.alloc(n, high=r.random() < 0.5)
            if off is None:
                assert p.stats()["largest_free"] < n
                continue
            assert off % 256 == 0 and off + n <= cap
            for o, m in live.items():
                assert off + n <= o or o + m <= off
            live[off] = n
        assert p.stats()["used"] == sum(live.values())
    for off in list(live):
        p.free(off)
    s = p.stats()
    assert s["used"] == 0 and s["front"] == 0 and s["largest_free"] == cap


# ---- the reserve's size from the environment (host only)
def _parse(text):
    import ctypes as C
    from cacti_amd import ffi
    out = C.c_uint64()
    rc = ffi.lib().cacti_parse_byte_size(text.encode(), C.byref(out))
    return None if rc else out.value


def test_parse_byte_size_vectors():
    """The examples the reference's parser documents (src/algo/str/parse_size.rs:126-129, 257-260)
    and the corners of its rules."""
    assert _parse("10 KB") == 10000 and _parse("20000") == 20000 and _parse("0.2 MiB") == 209715
    assert _parse("^_^") is None and _parse("") is None and _parse("KB") is None
    assert _parse("1 KB") == 1000 and _parse("1 KiB") == 1024 and _parse("1 MB") == 10 ** 6 and _parse("1 MiB") == 1 << 20
    assert _parse("128 B") == 128 and _parse("16 KiB") == 16384 and _parse("123k") == 123000 and _parse("123KB") == 123000
    assert _parse("16GiB") == 16 << 30 and _parse("16gib") == 16 << 30 and _parse("1_000_000") == 10 ** 6
    assert _parse("1.5e3") == 1500 and _parse("1e3 KB") == 10 ** 6 and _parse("25e-1") == 3      # 2.5 rounds half up
    assert _parse("1E") == 10 ** 18 and _parse("1Ei") == 1 << 60 and _parse("16E") == 16 * 10 ** 18
    assert _parse("19E") is None                                                               # beyond 64 bits
    assert _parse("18446744073709551615") == 2 ** 64 - 1 and _parse("18446744073709551616") is None
    assert _parse("0.0000000000000000000000000000000000000001") == 0 and _parse("1e-50") == 0
    assert _parse("1.2.3") is None and _parse("-5") is None and _parse("5 5") == 55


def test_vmem_soft_limit_rules():
    """NvGpuMemPool::new, src/pctx/nvgpu.rs:1434-1463: default 90.01 %, a decimal number is a fraction of the
    device, anything else a byte size, rounded down to 64 KiB."""
    import ctypes as C
    from cacti_amd import ffi

    def lim(text, avail, total):
        out = C.c_size_t()
        assert ffi.lib().cacti_vmem_soft_limit(None if text is None else text.encode(), avail, total, C.byref(out)) == 0
        return out.value

    total, avail = 288 * 10 ** 9, 287 * 10 ** 9
    dflt = ((total * 9001 + 9999) // 10000) >> 16 << 16
    assert lim(None, avail, total) == dflt and lim("", avail, total) == dflt and lim("lots", avail, total) == dflt
    assert lim("0.5", avail, total) == (total // 2) >> 16 << 16
    assert lim("16GiB", avail, total) == 16 << 30 and lim("16 GB", avail, total) == (16 * 10 ** 9) >> 16 << 16
    assert lim("17179869184B", avail, total) == 16 << 30
    full = (avail - (32 << 20)) >> 16 << 16
    assert lim("1.0", avail, total) == full and lim("17179869184", avail, total) == full        # a bare integer is a fraction
    assert lim("7", avail, total) == full and lim("-1", avail, total) == 0 and lim("nan", avail, total) == 0
    assert lim("1e-3", avail, total) == (total // 1000) >> 16 << 16
