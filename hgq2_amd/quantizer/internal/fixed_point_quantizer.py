"""Fixed-point quantizers with trainable bit-widths (KBI and KIF parametrisations).

Interface, variables (``_k`` uint8, ``_i``, ``_f`` / ``_b``, ``i_decay_speed``), state updates and
branch structure follow reference src/hgq/quantizer/internal/fixed_point_quantizer.py:
``FixedPointQuantizerBase`` (:34-150), ``FixedPointQuantizerKBI`` (:153-307),
``FixedPointQuantizerKIF`` (:310-459).  The arithmetic runs in the HIP kernels of
``libhgq_hip.so``: the raw variables are handed to the kernel, which rounds them, broadcasts
them, quantizes, and reduces the abs-max / bit-width gradients over the homogeneous axes.
"""

from __future__ import annotations

import numpy as np
import torch

from ... import _lib, ops
from ...constraints import Constraint, MinMax
from ...core import Constant as ConstantInit
from ...core import Initializer
from ...regularizers import Regularizer
from .base import TrainableQuantizerBase, bw_layout, numbers, round_conv  # noqa: F401


class FixedPointQuantizerBase(TrainableQuantizerBase):
    """Abstract base class for all fixed-point quantizers."""

    def __init__(self, **kwargs):
        super().__init__(**kwargs)
        self._seed_gen = None
        self._is_weight = False

    @property
    def round_mode(self) -> str:
        return self._round_mode

    @property
    def overflow_mode(self) -> str:
        return self._overflow_mode

    @property
    def seed_gen(self):
        return self._seed_gen

    def build(self, input_shape):
        if self.overflow_mode not in _lib.OVERFLOW_MODES:
            raise ValueError(f'unsupported overflow mode {self.overflow_mode}')
        if self.round_mode.startswith('S_'):  # reference :56-57
            from ..fixed_point_ops import SeedGenerator

            self._seed_gen = SeedGenerator(self._seed)
        if (self.round_mode[2:] if self.round_mode.startswith('S_') else self.round_mode) not in _lib.ROUND_MODES:
            raise ValueError(f'unsupported round mode {self.round_mode}')
        if self.overflow_mode == 'WRAP':
            init = self._i_decay_speed0
            self._i_decay_speed = self.add_weight(name='i_decay_speed', shape=(), initializer=init, trainable=False)
            # host copy of the variable for the launch arguments, refreshed when the variable is written
            self._decay_value = float(init.value) if isinstance(init, ConstantInit) else float(self._i_decay_speed)
            self._decay_version = self._i_decay_speed._version
        self._symmetric = self.overflow_mode.endswith('SYM')
        self.built = True

    @property
    def symmetric(self):
        return self._symmetric

    @property
    def i_decay_speed(self):
        return self._i_decay_speed

    @property
    def _decay_host(self) -> float:
        """``i_decay_speed`` as a host float (kernels take it as a launch argument): read back from the device only after
        the variable has been written (``assign``-style in-place writes and ``load_state_dict`` bump its version)."""
        v = self._i_decay_speed._version
        if v != self._decay_version:
            self._decay_value, self._decay_version = float(self._i_decay_speed), v
        return self._decay_value

    # ---- bit-width views (differentiable).  On the GPU one launch each way (`ops.qbits`); the torch
    # formula below is the same arithmetic as a chain of round / add / relu / cast launches.
    def _fused_bits(self, add_mode: int):
        kbi = not hasattr(self, '_f')
        fb = self._b if kbi else self._f
        if not (fb.is_cuda and fb.is_contiguous() and self._k.is_contiguous() and (kbi or self._i.is_contiguous())):
            return None
        from ... import ops

        return ops.qbits(self._k, None if kbi else self._i, fb, kbi, add_mode)

    @property
    def bits(self):
        fused = self._fused_bits(1 if self.overflow_mode == 'SAT' else 0)
        if fused is not None:
            return fused
        if self.overflow_mode != 'SAT':
            return self.b
        return self.b + self.k

    @property
    def fbits(self):
        fused = self._fused_bits(2 if self.overflow_mode == 'WRAP' else 1)
        if fused is not None:
            return fused
        b = self.b
        if self.overflow_mode == 'WRAP':
            return b + self.k * (b > 0).to(b.dtype)
        return b + self.k

    @property
    def min(self):
        if self.symmetric:
            return -self.k * (2.0**self.i - 2.0**-self.f)
        return -self.k * (2.0**self.i)

    @property
    def max(self):
        return 2.0**self.i - 2.0**-self.f

    @property
    def epsilon(self):
        return 2.0**-self.f

    def get_any_k(self, inputs):
        return self.bw_mapper.x_to_bw_sign(inputs)

    def __repr__(self) -> str:
        if not self.built:
            return f'{self.__class__.__name__}({self.round_mode}, {self.overflow_mode}, name={self.name}, built=False)'
        k, i, f = (t.detach().float().cpu().numpy() for t in (self.k, self.i, self.f))
        fmt = lambda a: f'{float(np.mean(a)):.2f}±{float(np.std(a)):.2f}'  # noqa: E731
        return (f'{self.__class__.__name__}(k={fmt(k)}, i={fmt(i)}, f={fmt(f)}, {self.round_mode}, '
                f'{self.overflow_mode}, name={self.name})')

    # ---- kernel plumbing
    _kbi = False

    def _third(self):
        return self._b if self._kbi else self._f

    def _mode(self, training: bool, overflow_mode: str | None = None) -> int:
        return _lib.mode_bits(self.round_mode, overflow_mode or self.overflow_mode, training=training, kbi=self._kbi,
                              round_params=True, symmetric=self._symmetric)

    def _operands(self, x):
        """Bit-width operands for the kernel and their layout relative to ``x``."""
        layout = bw_layout(self._i.shape, x.shape)
        if layout is not None:
            return self._k, self._i, self._third(), layout
        # broadcast pattern the kernels do not index: materialise (autograd sums the gradient back)
        shape = tuple(x.shape)
        k = torch.broadcast_to(self._k, shape).contiguous()
        i = torch.broadcast_to(self._i, shape).contiguous()
        t = torch.broadcast_to(self._third(), shape).contiguous()
        return k, i, t, (x.numel(), 1)

    @property
    def stochastic(self) -> bool:
        return self._seed_gen is not None

    def _quantize(self, x, mode: int, track: bool = False, stochastic: bool = False):
        """``stochastic``: this call is one of those the reference hands ``seed_gen`` to with training on (:147,:279,:404)."""
        k, i, t, (_, inner) = self._operands(x)
        if stochastic and self.stochastic and (mode & _lib.MODE_TRAINING):
            draw = self._seed_gen.next(x.device)  # on a GPU the counter sits in device memory: a recorded step draws anew per replay
            return ops.quantize_stochastic(x, k, i, t, mode, draw[0], draw[1], bw_inner=inner, track=track,
                                           base=draw[2] if len(draw) > 2 else None)
        return ops.quantize(x, k, i, t, mode, bw_inner=inner, track=track)

    def _constraint_bounds(self):
        c = self._i.constraint if hasattr(self._i, 'constraint') else None
        if c is None:
            return float('-inf'), float('inf')
        b = c.bounds()
        if b is None:
            raise NotImplementedError('only clip-type constraints are supported on the integer bits of a WRAP quantizer')
        return b

    def _track(self, amax, training, anyneg=None, clip=False):
        """Integer-bit tracking after a WRAP forward (reference :280-300, :406-422)."""
        tracing = not training
        lo, hi = self._constraint_bounds() if (clip or tracing) else (float('-inf'), float('inf'))
        mode = _lib.mode_bits(self.round_mode, self.overflow_mode, kbi=self._kbi, symmetric=self._symmetric,
                              tracing=tracing)
        if amax.numel() == 0 or amax.numel() % self._i.numel() != 0:  # one slice, or one per producing workgroup
            raise NotImplementedError('integer-bit tracking needs a bit-width layout the kernels can index')
        with torch.no_grad():
            ops.wrap_track_i_(amax, self._i.data.view(-1), self._third().data.view(-1), self._decay_host, mode, lo, hi,
                              anyneg=anyneg if (tracing and anyneg is not None) else None,
                              k_var=self._k.view(-1) if (tracing and anyneg is not None) else None)

    # ---- reference :142-150
    # (input, result) of this quantizer computed ahead of the layer call together with the other kernel / bias
    # quantizers of the model (quantizer/prefetch.py); used once, for that very input, in training mode
    _prefetched = None

    def _base_call(self, inputs, training: bool):
        pf, self._prefetched = self._prefetched, None
        if pf is not None and training and pf[0] is inputs:
            return pf[1]
        y, _, _ = self._quantize(inputs, self._mode(training), stochastic=training)
        return y

    def call(self, inputs, training=None):
        return self._base_call(inputs, training is True)


class FixedPointQuantizerKBI(FixedPointQuantizerBase):
    """Fixed-point quantizer parameterised by keep_negative, total bits and integer bits.

    Parameters: ``k0, b0, i0`` initial values (k not trained), ``round_mode`` in {'RND', 'TRN',
    'RND_CONV'}, ``overflow_mode`` in {'WRAP', 'SAT', 'SAT_SYM'}, ``bc / ic`` constraints,
    ``br / ir`` regularizers, ``i_decay_speed`` (WRAP only), ``is_weight``.
    """

    _kbi = True

    def __init__(self, k0, b0, i0, round_mode: str, overflow_mode: str, bc: Constraint | None = MinMax(0, 12),
                 ic: Constraint | None = None, br: Regularizer | None = None, ir: Regularizer | None = None,
                 i_decay_speed=float('inf'), is_weight: bool = False, **kwargs):
        super().__init__(**kwargs)
        if not isinstance(k0, Initializer) and not isinstance(b0, Initializer) and not isinstance(i0, Initializer):
            k0 = int(k0)
            assert k0 == 0 or k0 == 1, f'Invalid k0 value {k0}: must be 0 or 1.'
            assert b0 >= 0, f'Invalid b0 value {b0}: must be non-negative.'
        self._k0 = k0 if isinstance(k0, Initializer) else ConstantInit(float(k0))
        self._b0 = b0 if isinstance(b0, Initializer) else ConstantInit(float(b0))
        self._i0 = i0 if isinstance(i0, Initializer) else ConstantInit(float(i0))
        self._i_decay_speed0 = i_decay_speed if isinstance(i_decay_speed, Initializer) else ConstantInit(float(i_decay_speed))
        self._round_mode = round_mode.upper()
        self._overflow_mode = overflow_mode.upper()
        self.b_constraint, self.i_constraint = bc, ic
        self.b_regularizer, self.i_regularizer = br, ir
        self._is_weight = is_weight
        self.validate_config()

    def build(self, input_shape):
        bw_shape = self.bw_mapper.inference_weight_shape(input_shape)
        self._k = self.add_weight(name='k', shape=bw_shape, initializer=self._k0, trainable=False, dtype='uint8')
        self._b = self.add_weight(name='b', shape=bw_shape, initializer=self._b0, trainable=True,
                                  constraint=self.b_constraint, regularizer=self.b_regularizer)
        self._i = self.add_weight(name='i', shape=bw_shape, initializer=self._i0,
                                  trainable=self.overflow_mode != 'WRAP', constraint=self.i_constraint,
                                  regularizer=self.i_regularizer)
        super().build(input_shape)

    @property
    def k(self):
        return self._k.to(torch.float32)

    @property
    def b(self):
        return round_conv(self._b)

    @property
    def i(self):
        return round_conv(self._i)

    @property
    def f(self):
        return self.b - self.i

    @property
    def kif(self):
        k, b, i = self.k, self.b, self.i
        return k, i, b - i

    def validate_config(self):
        assert self.b_constraint is None or isinstance(self.b_constraint, Constraint)
        assert self.i_constraint is None or isinstance(self.i_constraint, Constraint)
        assert self.b_regularizer is None or isinstance(self.b_regularizer, Regularizer)
        assert self.i_regularizer is None or isinstance(self.i_regularizer, Regularizer)

    def call(self, inputs, training=None):
        if self.overflow_mode == 'WRAP' and self.trainable:
            if training or training == 'tracing':
                # the minimal integer bits come from the UN-rounded input (reference :281); `_i` is
                # assigned first and f = b - i is read afterwards, so rounding uses the new i
                is_training = bool(training)
                track_mode = self._mode(True) | _lib.MODE_TRACK_INPUT
                _, amax, _ = self._quantize(inputs.detach(), track_mode, track=True)
                self._track(amax, is_training, clip=True)
                y, _, neg = self._quantize(inputs, self._mode(True), track=not is_training, stochastic=training is True)
                if not is_training:
                    with torch.no_grad():
                        # the tracker arrives as one entry per bit-width entry or as [slices, entries]
                        seen = neg.view(-1, self._k.numel()).ne(0).any(0).view(self._k.shape)
                        new_k = seen & (torch.round(self._b) > 0)
                        self._k.copy_((self._k.bool() | new_k).to(torch.uint8))
                return y
            if self._is_weight and self.round_mode == 'RND':
                y, _, _ = self._quantize(inputs, self._mode(True))  # round only
                return y
        return self._base_call(inputs, training is True)


class FixedPointQuantizerKIF(FixedPointQuantizerBase):
    """Fixed-point quantizer parameterised by keep_negative, integer bits and fractional bits.

    Parameters: ``k0, i0, f0`` initial values (k not trained), ``round_mode``, ``overflow_mode``,
    ``ic / fc`` constraints, ``ir / fr`` regularizers, ``i_decay_speed`` (WRAP only), ``is_weight``.
    """

    _kbi = False

    def __init__(self, k0, i0, f0, round_mode: str, overflow_mode: str, ic: Constraint | None = None,
                 fc: Constraint | None = None, ir: Regularizer | None = None, fr: Regularizer | None = None,
                 i_decay_speed=float('inf'), is_weight: bool = False, **kwargs):
        super().__init__(**kwargs)
        if not isinstance(k0, Initializer) and not isinstance(i0, Initializer) and not isinstance(f0, Initializer):
            k0 = int(k0)
            assert k0 == 0 or k0 == 1, f'Invalid k0 value {k0}: must be 0 or 1.'
            assert i0 + f0 >= 0, f'Invalid i0+f0 value {i0 + f0}: must be non-negative.'
        self._k0 = k0 if isinstance(k0, Initializer) else ConstantInit(float(k0))
        self._i0 = i0 if isinstance(i0, Initializer) else ConstantInit(float(i0))
        self._f0 = f0 if isinstance(f0, Initializer) else ConstantInit(float(f0))
        self._i_decay_speed0 = i_decay_speed if isinstance(i_decay_speed, Initializer) else ConstantInit(float(i_decay_speed))
        self._round_mode = round_mode.upper()
        self._overflow_mode = overflow_mode.upper()
        self.i_constraint, self.f_constraint = ic, fc
        self.i_regularizer, self.f_regularizer = ir, fr
        self._is_weight = is_weight
        self.validate_config()

    def build(self, input_shape):
        bw_shape = self.bw_mapper.inference_weight_shape(input_shape)
        self._k = self.add_weight(name='k', shape=bw_shape, initializer=self._k0, trainable=False, dtype='uint8')
        self._i = self.add_weight(name='i', shape=bw_shape, initializer=self._i0,
                                  trainable=self.overflow_mode != 'WRAP', constraint=self.i_constraint,
                                  regularizer=self.i_regularizer)
        self._f = self.add_weight(name='f', shape=bw_shape, initializer=self._f0, trainable=True,
                                  constraint=self.f_constraint, regularizer=self.f_regularizer)
        super().build(input_shape)

    def wrap_training_fusable(self, training) -> bool:
        """True when the call reduces to "round with f, track max|.|" (reference :401-413), the
        form the dense kernel fuses into its operand load."""
        return self.overflow_mode == 'WRAP' and self.trainable and training is True and not self.stochastic

    def call(self, inputs, training=None):
        if self.overflow_mode == 'WRAP' and self.trainable:
            if training or training == 'tracing':
                is_training = bool(training)
                y, amax, neg = self._quantize(inputs, self._mode(True), track=True, stochastic=training is True)
                # training: the reference applies the constraint to a dead value (:411-412), so the
                # assigned value is unclipped; tracing clips before the max (:416-418)
                self._track(amax, is_training, anyneg=neg)
                return y
            if self._is_weight:
                y, _, _ = self._quantize(inputs, self._mode(True))
                return y
        return self._base_call(inputs, training is True)

    @property
    def k(self):
        return self._k.to(torch.float32)

    @property
    def b(self):
        return torch.relu(self.i + self.f)

    @property
    def i(self):
        ops.flush_tracks()  # an integer-bit update of this model call may still be queued
        return round_conv(self._i)

    @property
    def f(self):
        return round_conv(self._f)

    @property
    def kif(self):
        return self.k, self.i, self.f

    def validate_config(self):
        assert self.f_constraint is None or isinstance(self.f_constraint, Constraint)
        assert self.i_constraint is None or isinstance(self.i_constraint, Constraint)
        assert self.f_regularizer is None or isinstance(self.f_regularizer, Regularizer)
        assert self.i_regularizer is None or isinstance(self.i_regularizer, Regularizer)
