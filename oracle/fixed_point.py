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
* stochastic modes (``S_RND``, ``S_RND_CONV``): only the deterministic branch
  (``stochastic=False`` or ``training=False``) is restated.
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


class _RoundF(torch.autograd.Function):
    """Rounding to ``f`` fractional bits with the surrogate gradient (training)."""

    @staticmethod
    def forward(ctx, x, f, round_mode):
        scale = _pow2(f)
        xq = _round_scaled(x * scale, round_mode) / scale
        ctx.save_for_backward(xq - x)
        return xq

    @staticmethod
    def backward(ctx, g):
        (delta,) = ctx.saved_tensors
        return g, -LN2 * delta * g, None


def fixed_round(x, f, round_mode: str, training: bool):
    if training:
        return _RoundF.apply(x, f, round_mode)
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

    def round(self, x, f, stochastic=False, seed_gen=None, training=True):
        if stochastic:
            raise NotImplementedError('stochastic rounding is not restated by the oracle')
        return fixed_round(x, f, self.round_mode, training)

    def __call__(self, x, k, i, f, training=False, seed_gen=None):
        if self.stochastic and training:
            raise NotImplementedError('stochastic rounding is not restated by the oracle')
        xq = fixed_round(x, f, self.round_mode, bool(training))
        return _overflow(xq, k, i, f, self.overflow_mode, bool(training))


def get_fixed_quantizer(round_mode: str = 'TRN', overflow_mode: str = 'WRAP') -> FixedQuantizer:
    return FixedQuantizer(round_mode, overflow_mode)
