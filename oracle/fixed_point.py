"""Oracle (test infrastructure, never shipped): the stateless fixed-point quantizer.

The reference does not contain this arithmetic.  It imports it from the third-party
package ``quantizers`` (constraint ``quantizers>=1.2.2``, reference ``pyproject.toml:26``;
no lock file, so no exact pin exists):

    from quantizers.fixed_point._fixed_point_ops import _get_fixed_quantizer as get_fixed_quantizer
    from quantizers.fixed_point._fixed_point_ops import round_conv
    (reference src/hgq/quantizer/internal/fixed_point_quantizer.py:9-10)

That package is not in the reference tree and not installed, so this file restates
its published algorithm as eager fp32 torch-CPU ops, one op per ``keras.ops`` call,
in the order the formulas below give, so that every intermediate is the same IEEE-754
fp32 value the Keras/torch path produces:

    round   : xq = R(x * 2**f) / 2**f        R = floor(t)          TRN
                                             R = floor(t + 0.5)    RND
                                             R = round-half-even   RND_CONV
    WRAP    : training -> identity;  else  ((xq + k*2**i) mod 2**(i+k)) - k*2**i
    SAT     : clip(xq, -k*2**i,               2**i - 2**-f)
    SAT_SYM : clip(xq, -k*(2**i - 2**-f),     2**i - 2**-f)

Call sites in the reference that anchor the interface (``q(x,k,i,f,training,seed_gen)``,
``q.round(x,f,stochastic,seed_gen)``, ``q.stochastic``, ``q.round_mode``):
fixed_point_quantizer.py:58,147,279,288,295,304-305,404-405.

What pins what
--------------
* forward VALUES, all modes: pinned by ``oracle.exact`` (integer ap_fixed<W,I,Q,O>
  semantics, the behaviour the reference's tests demand of this path, reference
  tests/base.py:207-275) and by the closed-form range/step in
  fixed_point_quantizer.py:107-120.  See tests/test_oracle_pins.py.
* surrogate GRADIENTS: **parity unpinned**.  Nothing in the reference tree states
  them; only "a saturated weight receives no gradient" (reference tests/base.py:330).
  Restated here from the HGQ convention:
      d xq / d x = 1                    (straight-through)
      d xq / d f = -ln2 * (xq - x)      (the rounding error scales as 2**-f)
      clip: d/dx = 1 inside, 0 outside; the active bound receives the upstream
            gradient, and the bounds are differentiable functions of i and f:
            d max/d i = ln2*2**i, d max/d f = +ln2*2**-f, min = -k*2**i or -k*max.
  The clip part is additionally checked against finite differences of the bounds, and the
  rounding part against a numerical derivative of the stated error model
  (delta(f+h) = delta(f) * 2**-h); that the package uses this model stays unverifiable here.
* ``i`` is not clamped against ``-f`` inside the callable (any such clamp in the
  third-party package is unpinned; it can only matter where k+i+f <= 0, which the
  reference zeroes at inference, fixed_point_quantizer.py:148-149).
* stochastic modes (``S_RND``, ``S_RND_CONV``): the rule floor(x * 2^f + u), u uniform in [0, 1), in training and the
  deterministic counterpart otherwise is what the name and the call sites (fpq.py:279,404) fix; the package's own
  random stream (keras.random, backend-specific) cannot be matched, so the draw is this build's definition
  (``stochastic_uniform``: Philox4x32-10 keyed by the seed, counter = element block and call offset), pinned by the
  generator's published known-answer vectors and by the properties of stochastic rounding (neighbour values only,
  unbiased mean, reproducible per (seed, offset)).
"""

from __future__ import annotations

import math

import torch

LN2 = math.log(2.0)

ROUND_MODES = ('TRN', 'RND', 'RND_CONV')
OVERFLOW_MODES = ('WRAP', 'SAT', 'SAT_SYM')


def _pow2(e: torch.Tensor) -> torch.Tensor:
    """``2.0 ** e`` as keras.ops does it on the torch backend (fp32 pow)."""
    return torch.pow(torch.tensor(2.0, dtype=e.dtype), e)


def _round_scaled(t: torch.Tensor, round_mode: str) -> torch.Tensor:
    if round_mode == 'TRN':
        return torch.floor(t)
    if round_mode == 'RND':
        return torch.floor(t + 0.5)
    if round_mode == 'RND_CONV':
        return torch.round(t)  # half-to-even, same as keras.ops.round
    raise ValueError(f'unknown round mode {round_mode}')


class _RoundConv(torch.autograd.Function):
    """``round_conv``: round-half-even with a straight-through gradient.

    Identical local copy in the reference: src/hgq/quantizer/internal/base.py:19-28.
    """

    @staticmethod
    def forward(ctx, x):
        return torch.round(x)

    @staticmethod
    def backward(ctx, g):
        return g


def round_conv(x: torch.Tensor) -> torch.Tensor:
    return _RoundConv.apply(x)


def philox4x32_10(counter, key):
    """Philox4x32-10 (Salmon, Moraes, Dror, Shaw: "Parallel random numbers: as easy as 1, 2, 3", SC'11) on numpy uint64
    arrays holding 32-bit words: ``counter`` four arrays, ``key`` two; returns the four output words.  Pinned by the
    known-answer vectors of the authors' Random123 library (tests/test_oracle_pins.py)."""
    import numpy as np

    mask = np.uint64(0xFFFFFFFF)
    c = [np.asarray(v, dtype=np.uint64) & mask for v in counter]
    k = [np.asarray(v, dtype=np.uint64) & mask for v in key]
    for _ in range(10):
        p0, p1 = np.uint64(0xD2511F53) * c[0], np.uint64(0xCD9E8D57) * c[2]  # 32 x 32 -> 64 bits: no overflow in uint64
        c = [(p1 >> np.uint64(32)) ^ c[1] ^ k[0], p1 & mask, (p0 >> np.uint64(32)) ^ c[3] ^ k[1], p0 & mask]
        k = [(k[0] + np.uint64(0x9E3779B9)) & mask, (k[1] + np.uint64(0xBB67AE85)) & mask]
    return c


def stochastic_uniform(n: int, seed: int, offset: int) -> torch.Tensor:
    """The n uniform numbers in [0, 1) of one stochastic-rounding call: element e takes word e % 4 of the block with
    counter (e // 4, offset) under key ``seed``, top 24 bits.  (The draw this build defines; the reference's comes from
    keras.random and differs per backend.)"""
    import numpy as np

    blocks = np.arange((n + 3) // 4, dtype=np.uint64)
    off = np.full_like(blocks, offset)
    words = philox4x32_10([blocks, blocks >> np.uint64(32), off, off >> np.uint64(32)],
                          [np.uint64(seed), np.uint64(seed) >> np.uint64(32)])
    flat = np.stack(words, axis=1).reshape(-1)[:n]
    return torch.from_numpy(((flat >> np.uint64(8)).astype(np.float64) * 2.0**-24).astype(np.float32))


class SeedGenerator:
    """A seed and a call counter; ``next()`` names one call's draw."""

    def __init__(self, seed):
        self.seed, self.offset = int(seed), 0

    def next(self):
        self.offset += 1
        return self.seed, self.offset


def _draw(seed_gen):
    return seed_gen.next() if hasattr(seed_gen, 'next') else (int(seed_gen[0]), int(seed_gen[1]))


class _RoundF(torch.autograd.Function):
    """Rounding to ``f`` fractional bits with the surrogate gradient (training); with ``u`` the stochastic form
    floor(x * 2^f + u)."""

    @staticmethod
    def forward(ctx, x, f, round_mode, u=None):
        scale = _pow2(f)
        xq = (torch.floor(x * scale + u) if u is not None else _round_scaled(x * scale, round_mode)) / scale
        ctx.save_for_backward(xq - x)
        return xq

    @staticmethod
    def backward(ctx, g):
        (delta,) = ctx.saved_tensors
        return g, -LN2 * delta * g, None, None


def fixed_round(x, f, round_mode: str, training: bool, u=None):
    if training:
        return _RoundF.apply(x, f, round_mode, u)
    scale = _pow2(f)
    return _round_scaled(x * scale, round_mode) / scale


class _Clip(torch.autograd.Function):
    """clip(x, lo, hi); the active bound takes the upstream gradient."""

    @staticmethod
    def forward(ctx, x, lo, hi):
        over = x > hi
        under = x < lo
        ctx.save_for_backward(over, under)
        return torch.where(over, hi, torch.where(under, lo, x))

    @staticmethod
    def backward(ctx, g):
        over, under = ctx.saved_tensors
        zero = torch.zeros_like(g)
        return torch.where(over | under, zero, g), torch.where(under, g, zero), torch.where(over, g, zero)


def _overflow(xq, k, i, f, overflow_mode: str, training: bool):
    if overflow_mode == 'WRAP':
        if training:
            return xq
        bias = k * _pow2(i)
        return torch.remainder(xq + bias, _pow2(i + k)) - bias
    eps = _pow2(-f)
    hi = _pow2(i) - eps
    if overflow_mode == 'SAT':
        lo = -k * _pow2(i)
    elif overflow_mode == 'SAT_SYM':
        lo = -k * hi
    else:
        raise ValueError(f'unknown overflow mode {overflow_mode}')
    return _Clip.apply(xq, lo, hi)


class FixedQuantizer:
    """What ``get_fixed_quantizer(round_mode, overflow_mode)`` returns."""

    def __init__(self, round_mode: str = 'TRN', overflow_mode: str = 'WRAP'):
        round_mode = round_mode.upper()
        self.stochastic = round_mode.startswith('S_')
        if self.stochastic:
            round_mode = round_mode[2:]
        assert round_mode in ROUND_MODES, round_mode
        self.round_mode = round_mode
        self.overflow_mode = overflow_mode.upper()
        assert self.overflow_mode in OVERFLOW_MODES, overflow_mode

    def _uniform(self, x, seed_gen):
        seed, offset = _draw(seed_gen)
        return stochastic_uniform(x.numel(), seed, offset).view(x.shape)  # element order = row-major order of x

    def round(self, x, f, stochastic=False, seed_gen=None, training=True):
        return fixed_round(x, f, self.round_mode, training, self._uniform(x, seed_gen) if stochastic else None)

    def __call__(self, x, k, i, f, training=False, seed_gen=None):
        # a stochastic mode draws in training and is its deterministic counterpart otherwise
        u = self._uniform(x, seed_gen) if (self.stochastic and training) else None
        xq = fixed_round(x, f, self.round_mode, bool(training), u)
        return _overflow(xq, k, i, f, self.overflow_mode, bool(training))


def get_fixed_quantizer(round_mode: str = 'TRN', overflow_mode: str = 'WRAP') -> FixedQuantizer:
    return FixedQuantizer(round_mode, overflow_mode)
