"""The kernels divide many dividends by one divisor with a reciprocal that is refined once per divisor and two residual
corrections per quotient (csrc/common.hpp: make_divisor / divide) and claim the result equals the correctly rounded
fp32 quotient for their operand ranges.  Checked here in exact rational arithmetic, with the hardware's reciprocal
estimate modelled as the correctly rounded reciprocal moved by -1, 0 or +1 units in the last place (v_rcp_f32 is
specified to 1 ulp)."""
from fractions import Fraction

import numpy as np


def _round_f32(x: Fraction) -> np.float32:
    """round-to-nearest-even of an exact rational to fp32 (normal range)"""
    if x == 0:
        return np.float32(0.0)
    sign = -1 if x < 0 else 1
    x = abs(x)
    e = x.numerator.bit_length() - x.denominator.bit_length()
    if Fraction(2) ** e > x:
        e -= 1
    assert Fraction(2) ** e <= x < Fraction(2) ** (e + 1) and -126 <= e <= 127
    scaled = x / Fraction(2) ** (e - 23)            # in [2^23, 2^24)
    m, rem = divmod(scaled.numerator, scaled.denominator)
    twice = 2 * rem
    if twice > scaled.denominator or (twice == scaled.denominator and (m & 1)):
        m += 1
    return np.float32(sign * float(m) * 2.0 ** (e - 23))


def _fma(a, b, c):
    return _round_f32(Fraction(float(a)) * Fraction(float(b)) + Fraction(float(c)))


def _divide(n, d, ulp_shift):
    y0 = _round_f32(1 / Fraction(float(d)))
    if ulp_shift:
        y0 = np.nextafter(y0, np.float32(np.inf if ulp_shift > 0 else 0), dtype=np.float32)
    e = _fma(-d, y0, np.float32(1))
    y = _fma(e, y0, y0)
    q0 = _round_f32(Fraction(float(n)) * Fraction(float(y)))
    r0 = _fma(-d, q0, n)
    q1 = _fma(r0, y, q0)
    r1 = _fma(-d, q1, n)
    return _fma(r1, y, q1)


def _check(pairs):
    for n, d in pairs:
        want = _round_f32(Fraction(float(n)) / Fraction(float(d)))
        for shift in (-1, 0, 1):
            got = _divide(np.float32(n), np.float32(d), shift)
            assert got == want and np.signbit(got) == np.signbit(want), (float(n), float(d), shift, float(got), float(want))


def test_quantiser_ranges():
    """pre-pass: x a bf16/fp16 value of a row, d = max(absmax, 1e-5) / 127 or / 7, |x / d| <= 127 (or 7)"""
    rng = np.random.default_rng(1)
    pairs = []
    for _ in range(400):
        amax = np.float32(10.0 ** rng.uniform(-5, 4.8))
        for levels in (127.0, 7.0):
            d = np.float32(amax / np.float32(levels))
            xs = (rng.uniform(-1, 1, 3) * amax).astype(np.float32)
            xs = (xs.view(np.uint32) & 0xFFFF0000).view(np.float32)        # bf16-representable
            pairs += [(x, d) for x in xs]
            # dividends next to the rounding boundaries k + 1/2 of the quantiser
            k = rng.integers(0, int(levels))
            pairs.append((np.float32((k + 0.5) * float(d)), d))
    _check(pairs)


def test_index_ranges():
    """calibration: n = i - j and d = a row index, both integers in [0, 2^24] / [1, 2^24]"""
    rng = np.random.default_rng(2)
    pairs = [(np.float32(0), np.float32(1)), (np.float32(2 ** 24), np.float32(2 ** 24)), (np.float32(1), np.float32(2 ** 24))]
    for _ in range(500):
        d = int(rng.integers(1, 2 ** int(rng.integers(1, 25))))
        n = int(rng.integers(0, d + 1))
        pairs.append((np.float32(n), np.float32(d)))
    # bins are floor(num_bins * n / d): quotients just around k / num_bins
    for d in (199, 200, 3001, 65537, 131071):
        for k in (1, 7, 99, 150):
            n = (k * d) // 200
            pairs += [(np.float32(n), np.float32(d)), (np.float32(n + 1), np.float32(d))]
    _check(pairs)


def test_float_quantiser_ranges():
    """pre-pass with the e4m3 / e5m2 quantisers: d = max(absmax, 1e-5) / 448 or / 57344, |x / d| <= 448 (or 57344);
    dividends also next to the mantissa-rounding boundaries (1 + (k + 1/2) / 2^m) * 2^e of the float simulation"""
    rng = np.random.default_rng(3)
    pairs = []
    for _ in range(300):
        amax = np.float32(10.0 ** rng.uniform(-5, 4.8))
        for fmax, mbits in ((448.0, 3), (57344.0, 2)):
            d = np.float32(amax / np.float32(fmax))
            xs = (rng.uniform(-1, 1, 3) * amax).astype(np.float32)
            xs = (xs.view(np.uint32) & 0xFFFF0000).view(np.float32)
            pairs += [(x, d) for x in xs]
            k, e = int(rng.integers(0, 2 ** mbits)), int(rng.integers(-6, 8))
            pairs.append((np.float32((1 + (k + 0.5) / 2 ** mbits) * 2.0 ** e * float(d)), d))
    _check(pairs)


# ---- the integer counterpart: FastDiv (csrc/common.hpp) replaces x / d, d fixed per launch, by
# ((x * m >> 32) + x) >> s with s = ceil(log2 d), m = ceil(2^(32+s) / d) - 2^32, for x < 2^31.  Replayed here in
# Python integers (arbitrary precision), with the 32-bit wrap of the one addition the device code makes.
def _make_fastdiv(d):
    s = 0
    while (1 << s) < d:
        s += 1
    m = ((1 << (32 + s)) + d - 1) // d - (1 << 32)
    assert 0 <= m < (1 << 32), (d, m)
    return m, s


def _fastdiv(x, m, s):
    return ((((x * m) >> 32) + x) & 0xFFFFFFFF) >> s


def test_fastdiv_equals_integer_division_below_2_31():
    rng = np.random.default_rng(7)
    divisors = list(range(1, 70)) + [127, 128, 129, 448, 1000, 3584, 4608, 18944, 131072, 131073, 1048576, 2 ** 20 + 1,
                                     2 ** 30 - 1, 2 ** 30, 2 ** 30 + 1, 2 ** 31 - 1] + [int(v) for v in rng.integers(1, 2 ** 31, 200)]
    top = 2 ** 31 - 1
    for d in divisors:
        m, s = _make_fastdiv(d)
        xs = {0, 1, d - 1, d, d + 1, top, top - 1, top - d, (top // d) * d, (top // d) * d - 1}
        xs |= {int(k) * d + off for k in rng.integers(0, max(top // d, 1), 40) for off in (-1, 0, 1)}
        xs |= {int(v) for v in rng.integers(0, top + 1, 200)}
        for x in xs:
            if 0 <= x <= top:
                assert _fastdiv(x, m, s) == x // d, (x, d)
