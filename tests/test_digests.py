"""Numerical-health digests (NanCount, AbsLog2Hist8; src/thunk/op.rs:273-441): integer-exact.

CPU: the oracle's restatement (the reference's bit arithmetic, including its multiply-and-look-up
log2 of the subnormal mantissa) against an independent derivation from the value of every one of
the 65536 f16 bit patterns.  GPU: the HIP kernels against the oracle, bit for bit."""
import numpy as np
import pytest

from tests.util import rng


@pytest.fixture(scope="module")
def ops():
    import torch
    assert torch.cuda.is_available(), "these tests need the MI355X"
    from cacti_amd import ops as o
    return o


def all_patterns():
    return np.arange(65536, dtype=np.uint32).astype(np.uint16)


def bins_from_values(bits):
    """floor(log2 |x|) + 127 from the numeric value; 0 for zeros, 255 for inf / nan."""
    x = bits.view(np.float16).astype(np.float64)
    out = np.empty(bits.size, np.int64)
    fin = np.isfinite(x)
    out[~fin] = 255
    out[fin & (x == 0)] = 0
    nz = fin & (x != 0)
    _, e = np.frexp(np.abs(x[nz]))             # |x| = m 2^e with m in [0.5, 1)
    out[nz] = e - 1 + 127
    return out


def test_oracle_bins_match_the_values_of_all_f16_patterns(oracle):
    bits = all_patterns()
    want = bins_from_values(bits)
    got = np.array([oracle.abs_log2_bin(int(b)) for b in bits])
    assert np.array_equal(got, want)
    # subnormal, normal, zero and non-finite classes sit where the reference's comment-free
    # arithmetic puts them
    assert got[1] == 103 and got[0x3ff] == 112 and got[0x400] == 113 and got[0x7bff] == 142
    assert got[0] == 0 and got[0x8000] == 0 and got[0x7c00] == 255 and got[0xfe00] == 255


def test_oracle_histogram_and_nan_count(oracle):
    bits = all_patterns()
    h = oracle.abs_log2_hist8(bits.view(np.float16))
    assert h.dtype == np.int64 and h.shape == (256,) and h.sum() == 65536
    assert np.array_equal(h, np.bincount(bins_from_values(bits), minlength=256))
    assert oracle.nan_count(bits.view(np.float16)) == 2 * 1023        # both signs, mantissa 1..1023
    r = rng(7)
    x = (r.standard_normal(100003) * 0.02).astype(np.float16)
    assert oracle.nan_count(x) == 0
    assert np.array_equal(oracle.abs_log2_hist8(x), np.bincount(bins_from_values(x.view(np.uint16)), minlength=256))
    assert oracle.abs_log2_hist8(x[:0]).sum() == 0 and oracle.nan_count(x[:0]) == 0


def _cases():
    r = rng(11)
    w = (r.standard_normal((2048, 3200)) * 0.02).astype(np.float16)            # a weight matrix
    g = (r.standard_normal((1000, 333)) * 1e-6).astype(np.float16)             # subnormal-heavy, ragged size
    mixed = all_patterns().view(np.float16).copy()
    sprinkled = w[:64].copy().reshape(-1)
    sprinkled[r.integers(0, sprinkled.size, 500)] = np.float16("nan")
    sprinkled[r.integers(0, sprinkled.size, 300)] = np.float16("inf")
    sprinkled[r.integers(0, sprinkled.size, 300)] = np.float16(0)
    return {"weights": w, "tiny": g, "every pattern": mixed, "sprinkled": sprinkled,
            "one": w.reshape(-1)[:1].copy(), "seven": w.reshape(-1)[:7].copy(), "empty": w.reshape(-1)[:0].copy()}


@pytest.mark.gpu
@pytest.mark.parametrize("case", ["weights", "tiny", "every pattern", "sprinkled", "one", "seven", "empty"])
def test_digests_match_the_oracle_bit_for_bit(ops, oracle, case):
    import torch
    x = _cases()[case]
    print("digest", case, x.shape, flush=True)
    d = torch.from_numpy(x.view(np.int16)).cuda().view(torch.float16) if x.size else \
        torch.empty(0, dtype=torch.float16, device="cuda")
    h = ops.abs_log2_hist8(d).cpu().numpy()
    c = int(ops.nan_count(d).cpu())
    assert h.dtype == np.int64 and np.array_equal(h, oracle.abs_log2_hist8(x))
    assert c == oracle.nan_count(x)
    assert h.sum() == x.size


@pytest.mark.gpu
def test_digest_of_the_embedding_sized_tensor_is_consistent(ops):
    """At full size (32000 x 3200, no oracle run): the classes add up to the element count and the
    NaN count equals what torch sees; the outputs are overwritten, not accumulated."""
    import torch
    torch.manual_seed(0)
    x = (torch.randn(32000, 3200, device="cuda") * 0.02).half()
    x.view(-1)[::1000003] = float("nan")
    for _ in range(2):
        h = ops.abs_log2_hist8(x)
        c = ops.nan_count(x)
    assert int(h.sum()) == x.numel()
    assert int(c) == int(torch.isnan(x).sum())
    assert int(h[255]) == int((~torch.isfinite(x)).sum())


@pytest.mark.gpu
def test_batched_digests_match_the_oracle_bit_for_bit(ops, oracle):
    """All cases in one launch (ragged sizes, an empty tensor, tensors of several workgroups),
    twice into the same call pattern: the outputs are overwritten."""
    import torch
    cases = _cases()
    names = ["seven", "weights", "empty", "tiny", "every pattern", "one", "sprinkled", "weights"]
    ds = [torch.from_numpy(cases[k].view(np.int16)).cuda().view(torch.float16) if cases[k].size else
          torch.empty(0, dtype=torch.float16, device="cuda") for k in names]
    print("digest batch", [tuple(d.shape) for d in ds], flush=True)
    for _ in range(2):
        h, c = ops.digests(ds)
    h, c = h.cpu().numpy(), c.cpu().numpy()
    for i, k in enumerate(names):
        assert np.array_equal(h[i], oracle.abs_log2_hist8(cases[k])), k
        assert int(c[i]) == oracle.nan_count(cases[k]), k
    h0, c0 = ops.digests([])
    assert h0.shape == (0, 256) and c0.shape == (0,)
