"""Oracle pin (test infrastructure, never shipped): exact-arithmetic ``ap_fixed``.

Shares no code with ``oracle.fixed_point``.  Everything here is Python ``int`` /
``fractions.Fraction`` arithmetic, so there is no rounding of intermediates at all;
it states what a ``(k, i, f)`` fixed-point word *is*:

    word  = ap_fixed<W = k+i+f, I = k+i>  (ap_ufixed when k == 0)
    value = n * 2**-f,  n integer,  n in [-k*2**(i+f), 2**(i+f) - 1]

* quantisation mode:  AP_TRN  n = floor(x*2**f);  AP_RND  n = floor(x*2**f + 1/2);
  AP_RND_CONV  n = nearest, ties to even.
* overflow mode:  AP_WRAP  keep the low W bits (two's complement);  AP_SAT clamp to
  [n_min, n_max];  AP_SAT_SYM clamp to [-k*n_max, n_max].

This is the behaviour the reference's own tests demand of the path (bit-exact against
the hls4ml and alkaid fixed-point simulators, reference tests/base.py:207-275) and the
range / step the reference states in closed form
(src/hgq/quantizer/internal/fixed_point_quantizer.py:107-120).
"""

from __future__ import annotations

from fractions import Fraction
from math import floor


def exact_round(x: float, f: int, round_mode: str) -> int:
    """Integer ``n`` such that the rounded value is ``n * 2**-f``."""
    t = Fraction(x) * (Fraction(2) ** f)
    if round_mode == 'TRN':
        return floor(t)
    if round_mode == 'RND':
        return floor(t + Fraction(1, 2))
    if round_mode == 'RND_CONV':
        lo = floor(t)
        r = t - lo
        if r > Fraction(1, 2):
            return lo + 1
        if r < Fraction(1, 2):
            return lo
        return lo if lo % 2 == 0 else lo + 1
    raise ValueError(round_mode)


def exact_overflow(n: int, k: int, i: int, f: int, overflow_mode: str) -> int:
    """Apply the overflow mode to the integer ``n`` of a word with ``i+f`` magnitude bits."""
    bits = i + f
    assert bits >= 0 and k + bits > 0, 'not a valid fixed-point word'
    n_max = 2**bits - 1
    n_min = -k * 2**bits
    if overflow_mode == 'WRAP':
        mod = 2 ** (bits + k)
        return (n - n_min) % mod + n_min
    if overflow_mode == 'SAT':
        return min(max(n, n_min), n_max)
    if overflow_mode == 'SAT_SYM':
        return min(max(n, -k * n_max), n_max)
    raise ValueError(overflow_mode)


def exact_quantize(x: float, k: int, i: int, f: int, round_mode: str, overflow_mode: str) -> Fraction:
    n = exact_overflow(exact_round(x, f, round_mode), k, i, f, overflow_mode)
    return Fraction(n) / (Fraction(2) ** f)


def exact_minimal_i_given_xf(xr: float, f: int) -> int:
    """Least integer ``i`` with ``xr <= 2**i - 2**-f`` for ``xr >= 0``.

    This is the invariant behind ``ceil(log2(xr + 2**-f))``
    (reference fixed_point_quantizer.py:25-31, x >= 0 / symmetric branch).
    """
    assert xr >= 0
    target = Fraction(xr) + Fraction(2) ** (-f)
    i = -200
    while Fraction(2) ** i < target:
        i += 1
    return i
