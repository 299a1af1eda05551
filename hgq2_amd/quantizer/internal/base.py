"""Quantizer base classes and the bit-width mapper.

Mirrors reference src/hgq/quantizer/internal/base.py: ``round_conv`` (:19-28),
``BitwidthMapperBase`` (:31-48), ``check_axis`` (:51-68), ``TrainableQuantizerBase`` (:71-115),
``DummyQuantizer`` (:118-145), ``DefaultBitwidthMapper`` (:148-196).
"""

from __future__ import annotations

import functools
import math
from collections.abc import Sequence

import numpy as np
import torch

from ...core import Layer, epsilon

numbers = int | float | np.integer | np.floating


class _RoundConv(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x):
        return torch.round(x)

    @staticmethod
    def backward(ctx, g):
        return g


def round_conv(x):
    """Round half to even with a straight-through gradient."""
    return _RoundConv.apply(x)


class BitwidthMapperBase:
    """Maps a bit-width tensor onto the tensor it quantizes."""

    def bw_to_x(self, bw, x_shape):
        raise NotImplementedError

    def x_to_bw_absmax(self, x):
        raise NotImplementedError

    def inference_weight_shape(self, input_shape) -> tuple[int, ...]:
        raise NotImplementedError

    def get_config(self):
        raise NotImplementedError

    @classmethod
    def from_config(cls, config):
        return cls(**config)


def check_axis(axis: Sequence[int], ndim: int):
    """Axes counted from the front (negative ones wrap once); anything outside the rank is refused."""
    front = [a + ndim if a < 0 else a for a in axis]
    bad = [a for a in front if not 0 <= a < ndim]
    assert not bad, f'axes {bad} (of {list(axis)}) do not exist in a tensor of rank {ndim}'
    return front


class DefaultBitwidthMapper(BitwidthMapperBase):
    """Bit-widths are shared along the homogeneous axes and individual along the others."""

    def __init__(self, heterogeneous_axis=None, homogeneous_axis=None, **kwargs):
        # a restored mapper (_shape_inferenced) carries both lists; a new one names exactly one of them, the other follows
        self._shape_inferenced = bool(kwargs.pop('_shape_inferenced', False))
        if not self._shape_inferenced and (heterogeneous_axis is None) == (homogeneous_axis is None):
            raise AssertionError('give either heterogeneous_axis or homogeneous_axis, not both and not neither')
        self.heterogeneous_axis, self.homogeneous_axis = heterogeneous_axis, homogeneous_axis

    def inference_weight_shape(self, input_shape):
        rank = len(input_shape)
        if self.heterogeneous_axis is not None:
            own = sorted(check_axis(self.heterogeneous_axis, rank))
            shared = [a for a in range(rank) if a not in own]
            self.heterogeneous_axis, self.homogeneous_axis = tuple(check_axis(self.heterogeneous_axis, rank)), tuple(shared)
        elif self.homogeneous_axis is not None:
            shared = check_axis(self.homogeneous_axis, rank)
            self.homogeneous_axis = tuple(shared)
            self.heterogeneous_axis = tuple(a for a in range(rank) if a not in shared)
        # one entry per position along the axes with bit-widths of their own, a single one along the shared axes
        shape = [1] * rank
        for a in self.heterogeneous_axis:
            if input_shape[a] is None:
                raise AssertionError(f'axis {a} of {tuple(input_shape)} has no fixed size: it cannot carry bit-widths of its own')
            shape[a] = int(input_shape[a])
        self._shape_inferenced = True
        return tuple(shape)

    def bw_to_x(self, bw, x_shape):
        return torch.broadcast_to(bw, tuple(x_shape))

    def x_to_bw_absmax(self, x):
        if not self.homogeneous_axis:
            return torch.abs(x)
        return torch.amax(torch.abs(x), dim=tuple(self.homogeneous_axis), keepdim=True)

    def x_to_bw_sign(self, x):
        neg = x < 0
        for a in self.homogeneous_axis or ():
            neg = torch.any(neg, dim=a, keepdim=True)
        return neg

    def get_config(self):
        return dict(heterogeneous_axis=self.heterogeneous_axis, homogeneous_axis=self.homogeneous_axis,
                    _shape_inferenced=self._shape_inferenced)


def bw_layout(bw_shape, x_shape):
    """``(bw_size, bw_inner)`` such that element ``e`` of a contiguous tensor of ``x_shape`` uses
    bit-width entry ``(e // bw_inner) % bw_size`` of a contiguous tensor of ``bw_shape``, or
    ``None`` if the broadcast pattern is not of that form."""
    return _bw_layout(tuple(bw_shape), tuple(x_shape))


@functools.lru_cache(maxsize=4096)
def _bw_layout(bw_shape, x_shape):  # asked two dozen times per training step with the same few shape pairs
    if len(bw_shape) != len(x_shape):
        if math.prod(bw_shape) == 1:
            return 1, 1
        return None
    het = [a for a, (b, s) in enumerate(zip(bw_shape, x_shape)) if b != 1 or s == 1]
    real = [a for a in het if x_shape[a] != 1]
    if not real:
        return 1, 1
    first, last = real[0], real[-1]
    for a in range(first, last + 1):
        if bw_shape[a] != x_shape[a]:
            return None
    return math.prod(x_shape[first:last + 1]), math.prod(x_shape[last + 1:])


class TrainableQuantizerBase(Layer):
    """Abstract base class of all quantizers."""

    __dummy__ = False

    def __init__(self, **kwargs):
        homogeneous_axis = kwargs.pop('homogeneous_axis', ())
        heterogeneous_axis = kwargs.pop('heterogeneous_axis', None)
        bw_mapper = kwargs.pop('bw_mapper', None) or DefaultBitwidthMapper(heterogeneous_axis, homogeneous_axis)
        self._seed = kwargs.pop('seed', int(np.random.randint(0, 2**31)))
        super().__init__(**kwargs)
        self.bw_mapper = bw_mapper
        self.supports_masking = True

    def compute_output_shape(self, input_shape):
        return input_shape

    @property
    def bits(self):
        raise NotImplementedError

    @property
    def fbits(self):
        raise NotImplementedError

    @property
    def min(self):
        raise NotImplementedError

    @property
    def max(self):
        raise NotImplementedError

    @property
    def epsilon(self):
        raise NotImplementedError


class DummyQuantizer(TrainableQuantizerBase):
    """Identity; with it every Q-layer reduces to its plain parent."""

    __dummy__ = True

    def call(self, inputs, training=None):
        return inputs

    @property
    def bits(self):
        return torch.tensor(0.0)

    @property
    def fbits(self):
        return torch.tensor(0.0)

    @property
    def min(self):
        return -1e9

    @property
    def max(self):
        return 1e9

    @property
    def epsilon(self):
        return epsilon()
