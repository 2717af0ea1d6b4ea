"""Rebuilds ZM_POW64_LOG_TAB of ../zmath.hpp from its definition, with exact rational arithmetic.

The log table of glibc's double pow (from ARM's optimized routines, pow_log_data.c): the arguments
z in [0x1.69555p-1, 0x1.69555p0) fall into 128 subintervals of 2^45 consecutive doubles; for each,
1 / c is the multiple of 1/128 (below z = 1) or 1/256 (above) nearest to 1 / centre, so that z / c - 1
is exact in double; logc = log(c) rounded to a multiple of 2^-43, logctail = the nearest double of the rest.

    python3 pow64_table.py        prints the macro body: invc, logc, logctail per subinterval
"""
import struct
from fractions import Fraction

OFF = 0x3fe6955500000000


def as_double(bits):
    return struct.unpack("<d", struct.pack("<Q", bits))[0]


def bits(v):
    return "0x%016xull" % struct.unpack("<Q", struct.pack("<d", v))[0]


def log_fraction(c, terms=400):
    """log(c) for a rational c near 1 as 2 atanh((c - 1) / (c + 1)), far beyond double-double accuracy"""
    t = (c - 1) / (c + 1)
    t2, power, total = t * t, t, Fraction(0)
    for n in range(terms):
        total += power / (2 * n + 1)
        power *= t2
        if abs(power) < Fraction(1, 1 << 400):
            break
    return 2 * total


def round_half_even(x):
    f = x.numerator // x.denominator
    rest = x - f
    if rest > Fraction(1, 2) or (rest == Fraction(1, 2) and f % 2):
        f += 1
    return f


def main():
    print("ZM_POW64_LOG_TAB")
    for i in range(128):
        lo, hi = Fraction(as_double(OFF + (i << 45))), Fraction(as_double(OFF + ((i + 1) << 45)))
        centre = (lo + hi) / 2
        n = 128 if centre < 1 else 256
        invc = Fraction(round_half_even(n / centre), n)
        log_c = -log_fraction(invc) if invc != 1 else Fraction(0)
        logc = Fraction(round_half_even(log_c * (1 << 43)), 1 << 43)
        print("      " + ", ".join(bits(float(v)) for v in (invc, logc, log_c - logc)) + ",")


if __name__ == "__main__":
    main()
