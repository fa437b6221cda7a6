"""The fp8 path divides by the per-tensor scale as  (float)((double)x * RN64(1/(double)s)).
This must equal the IEEE fp32 quotient x / s bit for bit (whenever the quotient is a normal
number or overflows - smaller results all encode to fp8 zero).  numpy's float32 / float64
arithmetic is IEEE-correct, so the claim is checked here on the CPU over a few hundred
million operand pairs: random bit patterns, 16-bit-float operands, and quotients steered
onto fp32 rounding boundaries."""
import numpy as np
import pytest


def quotient_via_fp64(x, s):
    with np.errstate(all="ignore"):
        inv = np.float64(1.0) / s.astype(np.float64)
        return (x.astype(np.float64) * inv).astype(np.float32)


def check(x, s):
    with np.errstate(all="ignore"):
        want = x / s
    got = quotient_via_fp64(x, s)
    wb, gb = want.view(np.uint32), got.view(np.uint32)
    relevant = (np.abs(want) >= np.float32(2.0 ** -126)) | np.isinf(want)      # normal or overflowed
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    bad = relevant & ~nan & (wb != gb)
    assert not bad.any(), f"{int(bad.sum())} mismatches, e.g. x={x[bad][0]!r} s={s[bad][0]!r}"
    # below the normal range both are tiny: far inside the fp8 flush-to-zero zone (|q| <= 2^-10)
    small = ~relevant & ~nan
    assert (np.abs(got[small]) < 2.0 ** -100).all()


def test_random_bit_patterns():
    rng = np.random.default_rng(0)
    for _ in range(20):
        x = rng.integers(0, 2 ** 32, size=4_000_000, dtype=np.uint32).view(np.float32)
        s = rng.integers(0, 2 ** 32, size=4_000_000, dtype=np.uint32).view(np.float32)
        check(x, s)


@pytest.mark.parametrize("bits", [16, 8])
def test_sixteen_bit_operands_against_many_scales(bits):
    """bf16 (top 16 bits of an fp32) and half-like operands: every 16-bit pattern x 1500 random scales."""
    rng = np.random.default_rng(1)
    pats = (np.arange(65536, dtype=np.uint32) << 16).view(np.float32)
    if bits == 8:
        import torch
        pats = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.float16).float().numpy()
    for _ in range(15):
        s = np.exp(rng.uniform(np.log(1e-6), np.log(1e4), size=100)).astype(np.float32)
        x = np.tile(pats, 100)
        check(x, np.repeat(s, 65536))


def test_quotients_on_rounding_boundaries():
    """Choose x = RN(m * s) for fp32 midpoints m: the true quotient then sits as close to a
    rounding boundary as two fp32 operands allow."""
    rng = np.random.default_rng(2)
    for _ in range(10):
        s = np.exp(rng.uniform(np.log(1e-3), np.log(1e3), size=2_000_000)).astype(np.float32)
        q = np.exp(rng.uniform(np.log(1e-2), np.log(500.0), size=2_000_000)).astype(np.float32)
        m = q.astype(np.float64) + np.spacing(q).astype(np.float64) / 2         # midpoint above q (25 bits)
        x = (m * s.astype(np.float64)).astype(np.float32)
        for dx in (-1, 0, 1):
            check((x.view(np.int32) + dx).view(np.float32), s)


def test_degenerate_scales():
    x = np.array([0.0, -0.0, 1.0, -3.5, np.inf, -np.inf, np.nan, 1e-40, 3e38], dtype=np.float32)
    for sv in (0.0, -0.0, np.inf, -np.inf, np.nan, 1e-45, 3.4e38, -2.0):
        check(x, np.full_like(x, sv))
