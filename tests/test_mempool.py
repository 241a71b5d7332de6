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
