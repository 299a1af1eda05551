"""Quantized pooling layers (reference src/hgq/layers/pooling.py:23-315): the input quantizer
followed by the plain pooling; EBOPs ``sum(bits_in) * parallelization_factor / n_parallel``.
The 2-D window poolings run in the channels-last pooling kernels (``hgq_pool2d_fwd / _bwd``); the
global poolings are single reductions over the spatial axes."""

from __future__ import annotations

from math import prod

import torch

from .. import ops
from ..quantizer import QuantizerConfig
from .core.base import QLayerBaseSingleInput, scale_ebops


def _pair(v):
    return (int(v), int(v)) if isinstance(v, int) else tuple(int(t) for t in v)


class QBasePooling(QLayerBaseSingleInput):
    def __init__(self, *args, parallelization_factor=-1, iq_conf: QuantizerConfig | None = None,
                 oq_conf: QuantizerConfig | None = None, **kwargs):
        self.parallelization_factor = parallelization_factor
        super().__init__(*args, iq_conf=iq_conf, oq_conf=oq_conf, **kwargs)
        self.data_format = 'channels_last'

    def _compute_ebops(self, shape):
        bw_inp = self.iq.bits_(shape)
        return scale_ebops(torch.sum(bw_inp), self.parallelization_factor, self.n_parallel)

    def _ebops_loss_term(self, shape):
        # value, uint32 variable, loss term and the bit-width gradients in one launch where the quantizer allows it
        if self.enable_iq and self._beta is not None and self._beta.is_cuda and self.n_parallel:
            operand = self.iq.bits_operand(shape)
            n_cells = prod(int(s) for s in shape)
            if operand is not None and 0 < n_cells < 2**31 and operand[3] <= 30720:
                return ops.bits_ebops('sum', [operand], (n_cells, float(self.parallelization_factor), float(self.n_parallel),
                                                         float(self.ebops_factor)), self._beta, self._ebops)
        return super()._ebops_loss_term(shape)

    def pool(self, inputs):
        raise NotImplementedError

    def call(self, inputs, training=None):
        if self.enable_iq:
            inputs = self.iq(inputs, training=training)
        return self.pool(inputs)

    def build(self, input_shape):
        super().build(input_shape)
        out_shape = self.compute_output_shape(input_shape)
        self.n_parallel = None if None in out_shape[1:] else prod(out_shape[1:-1])
        if self.parallelization_factor <= 0:
            assert self.n_parallel is not None
            self.parallelization_factor = self.n_parallel


class _QWindowPooling2D(QBasePooling):
    _mode = 'max'

    def __init__(self, pool_size=(2, 2), strides=None, padding='valid', data_format=None, **kwargs):
        if data_format not in (None, 'channels_last'):
            raise NotImplementedError('pooling: channels_last only')
        super().__init__(**kwargs)
        self.pool_size = _pair(pool_size)
        self.strides = _pair(strides) if strides is not None else self.pool_size
        self.padding = padding.lower()
        assert self.padding in ('valid', 'same')

    def compute_output_shape(self, input_shape):
        out = [input_shape[0]]
        for n, p, s in zip(input_shape[1:3], self.pool_size, self.strides):
            out.append(None if n is None else (-(-n // s) if self.padding == 'same' else (n - p) // s + 1))
        return tuple(out) + (input_shape[3],)

    def pool(self, inputs):
        return ops.pool2d(inputs, self.pool_size, self.strides, self.padding, self._mode)

    def get_config(self):
        config = super().get_config()
        config.update({'pool_size': self.pool_size, 'strides': self.strides, 'padding': self.padding,
                       'parallelization_factor': self.parallelization_factor})
        return config


class QMaxPooling2D(_QWindowPooling2D):
    _mode = 'max'


class QAveragePooling2D(_QWindowPooling2D):
    _mode = 'avg'


class _QGlobalPooling(QBasePooling):
    _rank = 2
    _mode = 'avg'

    def __init__(self, data_format=None, keepdims=False, **kwargs):
        if data_format not in (None, 'channels_last'):
            raise NotImplementedError('pooling: channels_last only')
        super().__init__(**kwargs)
        self.keepdims = keepdims

    def get_config(self):
        config = super().get_config()
        config.update({'keepdims': self.keepdims, 'parallelization_factor': self.parallelization_factor})
        return config

    def compute_output_shape(self, input_shape):
        if self.keepdims:
            return (input_shape[0],) + (1,) * self._rank + (input_shape[-1],)
        return (input_shape[0], input_shape[-1])

    def pool(self, inputs):
        axes = tuple(range(1, 1 + self._rank))
        if self._mode == 'avg':
            if inputs.is_cuda and inputs.dtype == torch.float32 and inputs.dim() == self._rank + 2 and inputs.numel():
                # channels-last: the pooled axes are the middle ones and collapse into one
                y = ops.mean_mid(inputs.reshape(inputs.shape[0], -1, inputs.shape[-1]))
                return y.reshape(self.compute_output_shape(tuple(inputs.shape))) if self.keepdims else y
            return torch.mean(inputs, dim=axes, keepdim=self.keepdims)
        return torch.amax(inputs, dim=axes, keepdim=self.keepdims)


class QGlobalAveragePooling1D(_QGlobalPooling):
    _rank, _mode = 1, 'avg'


class QGlobalAveragePooling2D(_QGlobalPooling):
    _rank, _mode = 2, 'avg'


class QGlobalMaxPooling1D(_QGlobalPooling):
    _rank, _mode = 1, 'max'


class QGlobalMaxPooling2D(_QGlobalPooling):
    _rank, _mode = 2, 'max'
