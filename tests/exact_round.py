"""Correctly rounded sums by brute force over the whole value set of a 16-bit float format.

Independent of the oracle's bit tricks: every finite value of the format is
decoded to an exact Fraction, the exact sum is formed in rational arithmetic,
and the nearest representable value is found by bisection, ties going to the
value whose bit pattern is even.  Sums at or beyond max + ulp/2 overflow to Inf.
"""
import bisect
from fractions import Fraction

FORMATS = {"bf16": (8, 7), "f16": (5, 10)}          # (exponent bits, mantissa bits)


class Format:
    def __init__(self, name):
        self.name = name
        self.ebits, self.mbits = FORMATS[name]
        self.bias = (1 << (self.ebits - 1)) - 1
        self.emax = (1 << self.ebits) - 1
        self.inf = self.emax << self.mbits
        # positive finite values, by bit pattern 0 .. inf-1 (monotone increasing)
        self.pos = [self._decode_pos(b) for b in range(self.inf)]
        top = self.pos[-1]
        self.overflow = top + (top - self.pos[-2]) / 2           # >= this rounds to Inf

    def _decode_pos(self, b):
        e, m = b >> self.mbits, b & ((1 << self.mbits) - 1)
        if e == 0:
            return Fraction(m, 1 << self.mbits) * Fraction(2) ** (1 - self.bias)
        return (1 + Fraction(m, 1 << self.mbits)) * Fraction(2) ** (e - self.bias)

    def is_nan(self, b):
        return (b & 0x7FFF) > self.inf

    def is_inf(self, b):
        return (b & 0x7FFF) == self.inf

    def value(self, b):
        v = self.pos[b & 0x7FFF]
        return -v if b & 0x8000 else v

    def round_pos(self, x):
        """x >= 0 exact -> bit pattern of nearest value (ties to even pattern)."""
        if x >= self.overflow:
            return self.inf
        i = bisect.bisect_left(self.pos, x)
        if i < len(self.pos) and self.pos[i] == x:
            return i
        lo, hi = i - 1, i                        # pos[lo] < x < pos[hi]  (hi may be == inf index)
        hi_val = self.pos[hi] if hi < len(self.pos) else None
        if hi_val is None:                       # between max finite and overflow threshold
            return lo
        dlo, dhi = x - self.pos[lo], hi_val - x
        if dlo < dhi:
            return lo
        if dhi < dlo:
            return hi
        return lo if lo % 2 == 0 else hi

    def add(self, a, b):
        """Bit pattern of the correctly rounded a+b, or None when the result is NaN."""
        if self.is_nan(a) or self.is_nan(b):
            return None
        if self.is_inf(a) or self.is_inf(b):
            if self.is_inf(a) and self.is_inf(b):
                return a if (a & 0x8000) == (b & 0x8000) else None
            return a if self.is_inf(a) else b
        x = self.value(a) + self.value(b)
        if x == 0:
            # IEEE: exact zero sum is +0 unless both operands are -0 (round-to-nearest)
            both_neg_zero = (a == 0x8000 and b == 0x8000)
            return 0x8000 if both_neg_zero else 0x0000
        if x > 0:
            return self.round_pos(x)
        return 0x8000 | self.round_pos(-x)
