"""Exact-rational model of IEEE-754 arithmetic, used to pin the oracle.

Every operation is evaluated on fractions.Fraction (no rounding at all) and
then rounded once to the target binary format with round-to-nearest-even,
which is the definition of a correctly rounded IEEE operation.  Nothing here
uses numpy or C floating point for the arithmetic being checked, so it is an
independent statement of what "float32 division, then a separate float32 add,
then round-half-even" means.
"""
from fractions import Fraction
import math

FORMATS = {           # precision (bits incl. hidden), min normal exponent, max exponent
    "f32": (24, -126, 127),
    "f16": (11, -14, 15),
    "bf16": (8, -126, 127),
    "f64": (53, -1022, 1023),
}


def rn(x, fmt):
    """Round Fraction x to the nearest value of fmt (ties to even, gradual underflow)."""
    p, emin, emax = FORMATS[fmt]
    if x == 0:
        return Fraction(0)
    sign = -1 if x < 0 else 1
    a = abs(x)
    e = a.numerator.bit_length() - a.denominator.bit_length()
    if Fraction(2) ** e > a:
        e -= 1
    assert Fraction(2) ** e <= a < Fraction(2) ** (e + 1)
    e = max(e, emin)
    quantum = Fraction(2) ** (e - p + 1)
    n = a / quantum
    r = n.numerator // n.denominator
    rem = n - r
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and r % 2 == 1):
        r += 1
    out = r * quantum
    if out >= Fraction(2) ** (emax + 1):
        raise OverflowError("rounds to infinity")
    return sign * out


def rint_even(x):
    """Round Fraction to nearest integer, ties to even (torch.round / rintf)."""
    f = math.floor(x)
    rem = x - f
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and f % 2 == 1):
        f += 1
    return int(f)


def quantize_group_exact(values, bits, fmt="f32", scale_div="ieee"):
    """RTN of one group, following bitween/functional.py:22-29 operation by
    operation.  values: floats already representable in fmt.
    scale_div "ieee": (hi - lo) / Qmax is one correctly rounded division (eager
    torch on the CPU).  "reciprocal": eager torch on a GPU multiplies by the
    float32 reciprocal of a scalar divisor: r = RN32(1 / Qmax), then
    RN32((hi - lo) * r), then - for a 16-bit tensor - a second rounding to fmt.
    Returns (scale Fraction, zero_point int, q list[int])."""
    w = [Fraction(v) for v in values]
    for v in w:
        assert rn(v, fmt) == v, "input not representable in the math format"
    qmax = (1 << bits) - 1
    lo, hi = min(w), max(w)
    if scale_div == "ieee":
        scale = rn(rn(hi - lo, fmt) / qmax, fmt)
    else:
        assert scale_div == "reciprocal"
        op = "f64" if fmt == "f64" else "f32"                           # the type the multiplication is carried out in
        scale = rn(rn(rn(hi - lo, fmt) * rn(Fraction(1, qmax), op), op), fmt)
    import struct
    floor32 = Fraction(struct.unpack("f", struct.pack("f", 1e-8))[0])   # the float32 nearest 1e-8
    floor = rn(floor32, fmt) if fmt != "f32" else floor32               # 0 in f16
    if fmt == "f64":
        floor = Fraction(1e-8)                                          # the double nearest 1e-8
    scale = max(scale, floor)
    if scale == 0:
        raise ZeroDivisionError("scale rounds to zero in this format")
    zp = min(max(rint_even(rn(-lo / scale, fmt)), 0), qmax)
    q = []
    for v in w:
        t = rn(v / scale, fmt)
        t = rn(t + zp, fmt)
        q.append(min(max(rint_even(t), 0), qmax))
    return scale, zp, q


def pack_exact(q, bits):
    """Python-integer closed form of the packed words of one row:
    word j = sum_i q[j*vpi+i] << (i*bits), reinterpreted as signed 32-bit."""
    vpi = 32 // bits
    words = []
    for j in range(len(q) // vpi):
        u = 0
        for i in range(vpi):
            u |= int(q[j * vpi + i]) << (i * bits)
        words.append(u - (1 << 32) if u >= (1 << 31) else u)
    return words
