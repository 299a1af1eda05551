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


class SeedGenerator:
    """Stands in for ``keras.random.SeedGenerator`` (reference :56-57): a seed and a counter that advances with every
    draw.  ``next()`` names one call's draw as ``(seed, offset)``; the kernels derive every element's uniform number from
    that pair, so the backward pass recomputes it.  Keras' own stream is backend-specific and is not reproduced.

    On a GPU the counter lives in device memory: ``next(device)`` returns ``(seed, n, base)`` - the draw is
    ``(seed, base[0] + n)``, n counting the draws since ``base`` was last advanced - and
    ``hgq2_amd.ops.advance_seed_generators()`` (run by the outermost layer call of every step) adds the pending count to
    ``base`` in one launch.  The offsets are the ones the host counter would give (1, 2, 3, ...), but a step recorded into
    a HIP graph - the advance, then draws at fixed distances from ``base`` - draws anew on every replay.  ``offset`` keeps
    counting on the host; it does not see replays."""

    def __init__(self, seed: int | None = None):
        self.seed = int(seed if seed is not None else torch.seed()) & (2**63 - 1)
        self.offset = 0
        self._base = None  # int64[1] on the device the generator first drew on
        self._drawn = 0    # draws since `_base` was advanced

    def next(self, device=None):
        capturing = torch.cuda.is_available() and torch.cuda.is_current_stream_capturing()
        device = torch.device(device) if device is not None else None
        if device is not None and device.type == 'cuda':
            if self._base is None:
                if capturing:
                    # the counter would be created - and set - by a recorded launch, and set again on every replay
                    raise RuntimeError('stochastic rounding: run one step outside the capture first (it creates the draw counter on the device)')
                self._base = torch.tensor([self.offset], dtype=torch.int64, device=device)
            elif self._base.device != device:
                raise RuntimeError(f'this seed generator draws on {self._base.device}, not on {device}')
            self.offset += 1
            self._drawn += 1
            if not any(g is self for g in ops._SEED_PENDING):
                ops._SEED_PENDING.append(self)
            return self.seed, self._drawn, self._base
        if capturing:
            # the pair travels as a launch argument: a captured launch would repeat the same draw on every replay
            raise RuntimeError('stochastic rounding cannot be captured into a HIP graph with a host-side offset: pass the device to next()')
        self.offset += 1
        if self._base is not None:  # keep the device counter in step: base + pending = offset
            self._drawn += 1
            if not any(g is self for g in ops._SEED_PENDING):
                ops._SEED_PENDING.append(self)
        return self.seed, self.offset


def _draw(seed_gen, device=None):
    if isinstance(seed_gen, SeedGenerator):
        return seed_gen.next(device)
    if isinstance(seed_gen, (tuple, list)) and len(seed_gen) == 2:
        return int(seed_gen[0]), int(seed_gen[1])
    raise TypeError('stochastic rounding needs seed_gen: a SeedGenerator or a (seed, offset) pair')


class FixedQuantizer:
    def __init__(self, round_mode: str = 'TRN', overflow_mode: str = 'WRAP'):
        round_mode = round_mode.upper()
        self.stochastic = round_mode.startswith('S_')
        self.round_mode = round_mode[2:] if self.stochastic else round_mode
        self.overflow_mode = overflow_mode.upper()
        _lib.mode_bits(self.round_mode, self.overflow_mode)  # validates

    def _run(self, x, k, i, f, training, overflow_mode, draw=None):
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
        if draw is not None:
            y, _, _ = ops.quantize_stochastic(x.contiguous(), kc, ic, fc, mode, draw[0], draw[1], bw_inner=layout[1],
                                              base=draw[2] if len(draw) > 2 else None)
        else:
            y, _, _ = ops.quantize(x.contiguous(), kc, ic, fc, mode, bw_inner=layout[1])
        return y

    def __call__(self, x, k, i, f, training=False, seed_gen=None):
        # stochastic modes draw in training and are their deterministic counterparts otherwise.
        # inference mode: entries with k+i+f <= 0 (empty words) come out as zero, which is what
        # the reference applies around the callable (fixed_point_quantizer.py:148-149)
        draw = _draw(seed_gen, x.device) if (self.stochastic and training) else None
        return self._run(x, k, i, f, training, self.overflow_mode, draw)

    def round(self, x, f, stochastic=False, seed_gen=None):
        # rounding only = the WRAP training branch; k and i are not read there (0-dim constants, nothing expanded)
        one = torch.ones((), dtype=x.dtype, device=x.device)
        zero = torch.zeros((), dtype=x.dtype, device=x.device)
        return self._run(x, one, zero, f, True, 'WRAP', _draw(seed_gen, x.device) if stochastic else None)


def get_fixed_quantizer(round_mode: str = 'TRN', overflow_mode: str = 'WRAP') -> FixedQuantizer:
    return FixedQuantizer(round_mode, overflow_mode)


_get_fixed_quantizer = get_fixed_quantizer
