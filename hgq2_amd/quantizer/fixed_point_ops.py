"""The stateless fixed-point quantizer callable, backed by the HIP kernels.

Drop-in for what the reference imports as
``from quantizers.fixed_point._fixed_point_ops import _get_fixed_quantizer as get_fixed_quantizer``
and ``round_conv`` (reference src/hgq/quantizer/internal/fixed_point_quantizer.py:9-10):
``q = get_fixed_quantizer(round_mode, overflow_mode)``; ``q(x, k, i, f, training, seed_gen)``;
``q.round(x, f, stochastic, seed_gen)``; attributes ``q.stochastic`` and ``q.round_mode``.
``k, i, f`` have the shape of ``x`` (they may be stride-0 broadcasts of smaller tensors, which
are recognised so that nothing is materialised) and must hold integer values.
"""

from __future__ import annotations

import torch

from .. import _lib, ops
from .internal.base import bw_layout, round_conv  # noqa: F401  (re-exported)


def _compact(t: torch.Tensor) -> torch.Tensor:
    """Undo a ``broadcast_to``: keep one entry along every stride-0 axis."""
    for d in range(t.dim()):
        if t.shape[d] > 1 and t.stride(d) == 0:
            t = t.narrow(d, 0, 1)
    return t


class FixedQuantizer:
    def __init__(self, round_mode: str = 'TRN', overflow_mode: str = 'WRAP'):
        round_mode = round_mode.upper()
        self.stochastic = round_mode.startswith('S_')
        self.round_mode = round_mode[2:] if self.stochastic else round_mode
        self.overflow_mode = overflow_mode.upper()
        _lib.mode_bits(self.round_mode, self.overflow_mode)  # validates

    def _run(self, x, k, i, f, training, overflow_mode):
        shape = tuple(x.shape)
        small = []
        for t in (k, i, f):
            t = torch.as_tensor(t, dtype=x.dtype, device=x.device)
            if tuple(t.shape) != shape:
                t = torch.broadcast_to(t, shape)
            small.append(_compact(t))
        # the three operands may broadcast along different axes (``round`` passes constants for k and i): the
        # bit-width block is the smallest shape that holds all of them
        bw_shape = tuple(max(dims) for dims in zip(*(t.shape for t in small))) if shape else ()
        layout = bw_layout(bw_shape, shape)
        if layout is None:  # a broadcast pattern the kernels do not index: per-element operands
            bw_shape, layout = shape, (x.numel(), 1)
        kc, ic, fc = (t.expand(bw_shape).contiguous() for t in small)
        mode = _lib.mode_bits(self.round_mode, overflow_mode, training=bool(training))
        y, _, _ = ops.quantize(x.contiguous(), kc, ic, fc, mode, bw_inner=layout[1])
        return y

    def __call__(self, x, k, i, f, training=False, seed_gen=None):
        if self.stochastic and training:
            raise NotImplementedError('stochastic rounding is not part of this build')
        # inference mode: entries with k+i+f <= 0 (empty words) come out as zero, which is what
        # the reference applies around the callable (fixed_point_quantizer.py:148-149)
        return self._run(x, k, i, f, training, self.overflow_mode)

    def round(self, x, f, stochastic=False, seed_gen=None):
        if stochastic:
            raise NotImplementedError('stochastic rounding is not part of this build')
        # rounding only = the WRAP training branch; k and i are not read there (0-dim constants, nothing expanded)
        one = torch.ones((), dtype=x.dtype, device=x.device)
        zero = torch.zeros((), dtype=x.dtype, device=x.device)
        return self._run(x, one, zero, f, True, 'WRAP')


def get_fixed_quantizer(round_mode: str = 'TRN', overflow_mode: str = 'WRAP') -> FixedQuantizer:
    return FixedQuantizer(round_mode, overflow_mode)


_get_fixed_quantizer = get_fixed_quantizer
