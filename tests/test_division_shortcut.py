"""The normalisation kernels divide a whole row by one scalar s as
float(double(y) * (1.0 / double(s))) (hc_amd/csrc/kernels/map.hip,
layer_norm_rows) and claim that this is the correctly rounded fp32 quotient
y / s whenever the quotient is a normal number.  The claim is arithmetic, so it
is checked here on the CPU with NumPy's IEEE division as the judge: random
pairs, every finite fp16 dividend against random divisors (the fp16 RMS norm),
and pairs built to sit next to a rounding boundary."""

import numpy as np

TINY = np.float32(1.17549435e-38)


def _shortcut(y, s):
    with np.errstate(all="ignore"):
        return (y.astype(np.float64) * (1.0 / s.astype(np.float64))).astype(np.float32)


def _check(y, s):
    with np.errstate(all="ignore"):
        want = y / s
    got = _shortcut(y, s)
    normal = np.isfinite(want) & (np.abs(want) >= TINY)
    assert normal.any()
    np.testing.assert_array_equal(got[normal].view(np.uint32), want[normal].view(np.uint32))
    # what the kernel sends the long way is exactly the rest: zero or subnormal quotients of
    # non-zero dividends, and quotients that are not finite, are recognised by their exponent
    ex = (got.view(np.uint32) >> 23) & 255
    long_way = (ex == 255) | ((ex == 0) & (y != 0))
    assert not (long_way & normal).any()
    assert (long_way | normal | (y == 0)).all()


def test_random_pairs():
    rng = np.random.default_rng(5)
    for scale in (1.0, 1e-30, 1e30):
        y = (rng.standard_normal(4_000_000) * scale).astype(np.float32)
        s = np.abs(rng.standard_normal(4_000_000)).astype(np.float32) + np.float32(1e-3)
        _check(y, s)
    bits = rng.integers(0x00800000, 0x7f800000, 4_000_000, dtype=np.uint32)
    y = bits.view(np.float32) * rng.choice(np.array([-1, 1], np.float32), bits.size)
    s = rng.integers(0x20000000, 0x5f000000, bits.size, dtype=np.uint32).view(np.float32)
    _check(y, s)


def test_every_fp16_dividend():
    rng = np.random.default_rng(6)
    h = np.arange(1 << 16, dtype=np.uint16).view(np.float16)
    y = h[np.isfinite(h)].astype(np.float32)
    for _ in range(40):
        s = np.full(y.shape, np.abs(rng.standard_normal()) * 10.0 ** rng.uniform(-6, 6), np.float32)
        _check(y, s)


def test_quotients_next_to_a_rounding_boundary():
    # y = round(m * s) for m half-way between two fp32 values: y / s then lies as close to
    # the midpoint m as the operands allow
    rng = np.random.default_rng(7)
    n = 2_000_000
    s = (1.0 + rng.random(n)).astype(np.float32)
    q = rng.integers(1 << 23, 1 << 24, n).astype(np.float64)
    mid = (q + 0.5) * 2.0 ** -23
    for nudge in (0, 1, -1):
        y = (mid * s.astype(np.float64)).astype(np.float32)
        y = (y.view(np.uint32).astype(np.int64) + nudge).astype(np.uint32).view(np.float32)
        _check(y, s)
    # divisors with the largest significands (where the reciprocal is least accurate)
    s = (np.uint32(0x3fffff00) + rng.integers(0, 256, n, dtype=np.uint32)).view(np.float32)
    y = (rng.random(n) + 1.0).astype(np.float32)
    _check(y, s)
