"""CPU: the split of a float into three bfloat16 pieces (hi, mid, lo), emulated in numpy exactly as
`split_bf16x3_kernel` and the piece-storing epilogues compute it (truncate to the upper 16 bits of
the float's bit pattern, subtract, truncate, subtract), over the magnitudes where it is exact and
the ones where it is not."""
import numpy as np


def split3(x):
    x = np.asarray(x, dtype=np.float32)
    xb = x.view(np.uint32)
    hb = xb & np.uint32(0xFFFF0000)
    finite = (xb & np.uint32(0x7F800000)) != np.uint32(0x7F800000)
    with np.errstate(invalid="ignore"):
        r1 = np.where(finite, x - hb.view(np.float32), np.float32(0)).astype(np.float32)
    mb = r1.view(np.uint32) & np.uint32(0xFFFF0000)
    r2 = (r1 - mb.view(np.float32)).astype(np.float32)
    lb = r2.view(np.uint32) & np.uint32(0xFFFF0000)
    return hb.view(np.float32), mb.view(np.float32), lb.view(np.float32)


def flush(p):
    """A matrix unit that reads bfloat16 denormals as zero."""
    return np.where(np.abs(p) < np.float32(2.0 ** -126), np.float32(0), p)


def random_floats(rng, lo_exp, hi_exp, n):
    mant = rng.integers(0, 1 << 23, size=n, dtype=np.uint32)
    exp = rng.integers(lo_exp + 127, hi_exp + 128, size=n, dtype=np.uint32)
    sign = rng.integers(0, 2, size=n, dtype=np.uint32)
    return ((sign << np.uint32(31)) | (exp << np.uint32(23)) | mant).view(np.float32)


def test_exact_from_two_to_the_minus_102_upwards():
    """|x| >= 2^-102: the lowest piece is at least 2^-126, so all three pieces are normal bfloat16
    values (or zero) and add up to x exactly, also for a unit that flushes denormals."""
    rng = np.random.default_rng(7)
    x = random_floats(rng, -102, 127, 200000)
    hi, mid, lo = split3(x)
    total = hi.astype(np.float64) + mid.astype(np.float64) + lo.astype(np.float64)
    assert np.array_equal(total, x.astype(np.float64))
    for p in (hi, mid, lo):
        assert np.array_equal(flush(p), p)
        assert np.array_equal(p.view(np.uint32) & np.uint32(0xFFFF), np.zeros_like(p.view(np.uint32)))


def test_bounded_below_that():
    """Smaller magnitudes: the remainders become fp32 denormals whose upper 16 bits no longer hold
    all their digits. Without flushing, what is dropped lies below 2^-133 (the last place of a
    bfloat16 denormal) and only for |x| < 2^-110; with flushing a piece below 2^-126 is lost whole:
    the sum is then off by less than 2^-125 in absolute terms. Either is far below anything an fp32
    sum of products of ordinary magnitudes resolves."""
    rng = np.random.default_rng(8)
    x = random_floats(rng, -126, -103, 200000)
    hi, mid, lo = split3(x)
    exact = x.astype(np.float64)
    err = np.abs(hi.astype(np.float64) + mid.astype(np.float64) + lo.astype(np.float64) - exact)
    assert err.max() < 2.0 ** -133
    assert (err[np.abs(x) >= np.float32(2.0 ** -110)] == 0).all()
    errf = np.abs(sum(flush(p).astype(np.float64) for p in (hi, mid, lo)) - exact)
    assert errf.max() < 2.0 ** -125
    # fp32 denormal inputs: hi alone is already a truncated denormal
    d = (rng.integers(1, 1 << 23, size=1000, dtype=np.uint32)).view(np.float32)
    hi, mid, lo = split3(d)
    assert np.abs(hi.astype(np.float64) + mid.astype(np.float64) + lo.astype(np.float64) - d.astype(np.float64)).max() < 2.0 ** -133


def test_specials_stay_in_the_first_piece():
    x = np.array([np.inf, -np.inf, np.nan, 0.0, -0.0, 3.4028235e38], dtype=np.float32)
    hi, mid, lo = split3(x)
    assert np.isinf(hi[0]) and np.isinf(hi[1]) and np.isnan(hi[2])
    assert (mid[:5] == 0).all() and (lo[:5] == 0).all()
    assert hi[5].astype(np.float64) + mid[5].astype(np.float64) + lo[5].astype(np.float64) == np.float64(x[5])
