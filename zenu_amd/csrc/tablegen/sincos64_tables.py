"""Rebuilds ZM_SINCOS64_TAB and ZM_TOVERP_TAB of ../zmath.hpp from their definitions, with exact rational arithmetic.

ZM_SINCOS64_TAB: for k = 0 .. 110 the four doubles sin(k/128), its remainder, cos(k/128), its remainder --
each value as the nearest double and the nearest double of what is left (the table of the double sin / cos
of the IBM Accurate Mathematical Library, which glibc ships as s_sin.c, is defined that way).
ZM_TOVERP_TAB: 2/pi in 75 pieces of 24 bits, as doubles (branred.c's table).

    python3 sincos64_tables.py        prints both macro bodies
"""
import struct
from fractions import Fraction


def sin_cos(x, terms=70):
    s, c, t = Fraction(0), Fraction(0), Fraction(1)
    for n in range(terms):                      # t = x^n / n!
        if n % 2 == 0:
            c += t if (n // 2) % 2 == 0 else -t
        else:
            s += t if (n // 2) % 2 == 0 else -t
        t = t * x / (n + 1)
    return s, c


def two_doubles(v):
    hi = float(v)                               # float(Fraction) rounds to nearest
    return hi, float(v - Fraction(hi))


def bits(v):
    return "0x%016xull" % struct.unpack("<Q", struct.pack("<d", v))[0]


def arctan_inverse(n, digits):
    one = 10 ** digits
    x = one // n
    total, n2, k, sign = x, n * n, 1, 1
    while x:
        x //= n2
        k += 2
        sign = -sign
        total += sign * (x // k)
    return total


def main():
    values = []
    for k in range(111):
        s, c = sin_cos(Fraction(k, 128))
        values += [*two_doubles(s), *two_doubles(c)]
    print("ZM_SINCOS64_TAB")
    for i in range(0, len(values), 4):
        print("      " + ", ".join(bits(v) for v in values[i:i + 4]) + ",")
    digits = 700
    pi = Fraction(4 * (4 * arctan_inverse(5, digits) - arctan_inverse(239, digits)), 10 ** digits)   # Machin
    t = 2 / pi
    pieces = []
    for _ in range(75):
        t *= 1 << 24
        pieces.append(int(t))
        t -= int(t)
    print("ZM_TOVERP_TAB")
    for i in range(0, 75, 8):
        print("      " + ", ".join("%d.0" % p for p in pieces[i:i + 8]) + ",")


if __name__ == "__main__":
    main()
