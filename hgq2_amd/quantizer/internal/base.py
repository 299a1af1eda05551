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
    axis = [a if a >= 0 else a + ndim for a in axis]
    assert all(0 <= a < ndim for a in axis), f'Invalid axis {axis} for shape {ndim}.'
    return axis


class DefaultBitwidthMapper(BitwidthMapperBase):
    """Bit-widths are shared along the homogeneous axes and individual along the others."""

    def __init__(self, heterogeneous_axis=None, homogeneous_axis=None, **kwargs):
        _shape_inferenced = kwargs.pop('_shape_inferenced', False)
        if not _shape_inferenced:
            assert (heterogeneous_axis is None) ^ (homogeneous_axis is None), (
                'Only one of quantize_dims and skip_dims can be specified.'
            )
        self.heterogeneous_axis = heterogeneous_axis
        self.homogeneous_axis = homogeneous_axis
        self._shape_inferenced = _shape_inferenced

    def inference_weight_shape(self, input_shape):
        n = len(input_shape)
        axis = np.arange(n)
        if self.heterogeneous_axis is not None:
            self.heterogeneous_axis = tuple(check_axis(self.heterogeneous_axis, n))
            self.homogeneous_axis = tuple(int(a) for a in np.setdiff1d(axis, self.heterogeneous_axis))
        elif self.homogeneous_axis is not None:
            self.homogeneous_axis = tuple(check_axis(self.homogeneous_axis, n))
            self.heterogeneous_axis = tuple(int(a) for a in np.setdiff1d(axis, self.homogeneous_axis))
        weight_shape = [1] * n
        for i in self.heterogeneous_axis:
            assert input_shape[i] is not None, (
                f'Unable to heterogeneously quantize axis {i} with unknown shape. Input shape: {input_shape}.'
            )
            weight_shape[i] = int(input_shape[i])
        self._shape_inferenced = True
        return tuple(weight_shape)

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
