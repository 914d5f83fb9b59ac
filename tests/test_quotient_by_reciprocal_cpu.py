"""The quantisers divide by the scale as x * r plus two remainder corrections (r = RN(1 / s)).
This checks the arithmetic itself, in exact rational numbers, against the correctly rounded quotient:
bf16 numerators of every exponent the path can see, the scales of the benchmark configurations, random
scales, and scales next to powers of two.  (The GPU tests check the kernels bit for bit against
torch's casts on all 65 536 bf16 patterns for a list of scales; this one covers the scales in between.)"""
from fractions import Fraction
import random
import struct


def rn32(q: Fraction) -> Fraction:
    """Round a rational to the nearest fp32 value (ties to even); normal range only."""
    if q == 0:
        return q
    sign = -1 if q < 0 else 1
    a = abs(q)
    e = a.numerator.bit_length() - a.denominator.bit_length()
    if Fraction(2) ** e > a:
        e -= 1
    assert -126 <= e <= 127
    ulp = Fraction(2) ** (e - 23)
    n = a / ulp                      # in [2^23, 2^24)
    fl = n.numerator // n.denominator
    rem = n - fl
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and fl % 2 == 1):
        fl += 1
    return sign * fl * ulp


def f32(bits: int) -> Fraction:
    return Fraction(struct.unpack("<f", struct.pack("<I", bits))[0])


def quotient_fast(x: Fraction, s: Fraction) -> Fraction:
    r = rn32(1 / s)
    q = rn32(x * r)                  # may be more than one unit in the last place off
    q = rn32(q + rn32(x - q * s) * r)
    rem = x - q * s                  # the second remainder must be exact in fp32 (the kernel's FMA rounds it)
    assert rn32(rem) == rem
    return rn32(q + rem * r)


def scales():
    rng = random.Random(7)
    yield from (Fraction(1), f32(0x3D000000), f32(struct.unpack("<I", struct.pack("<f", 100 / 448))[0]),
                f32(struct.unpack("<I", struct.pack("<f", 1.6 / 448))[0]), f32(struct.unpack("<I", struct.pack("<f", 0.75 / 448))[0]))
    for _ in range(150):
        yield f32((rng.randrange(100, 150) << 23) | rng.randrange(1 << 23))
    for e in (110, 127, 130):
        for m in (0, 1, 2, 0x7ffffe, 0x400000, 0x3fffff):      # all-ones significands take the kernel's IEEE path
            yield f32((e << 23) | m)


def test_corrected_quotient_is_correctly_rounded():
    rng = random.Random(11)
    checked = 0
    for s in scales():
        for _ in range(120):
            bits = (rng.randrange(90, 160) << 7 | rng.randrange(128)) << 16      # a bf16 number as fp32 bits
            if rng.random() < 0.5:
                bits |= 0x80000000
            x = f32(bits)
            want = rn32(x / s)
            assert quotient_fast(x, s) == want, (float(x), float(s))
            checked += 1
    assert checked > 15000
