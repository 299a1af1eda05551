"""The handful of plain (un-quantized) host-framework names the reference's examples use next to the quantized
layers (reference README.md:57-67: ``keras.Sequential``, ``keras.layers.MaxPooling2D``, ``keras.layers.Flatten``),
on the torch-native layer runtime of ``hgq2_amd.core``.  With ``import hgq2_amd.host as keras`` the README example
runs as written.  Tensors are channels-last, as in Keras."""

from __future__ import annotations

from types import SimpleNamespace

import torch

from . import ops
from .core import Layer, Sequential  # noqa: F401  (Sequential is part of this module's surface)


def _pair(v):
    return (int(v), int(v)) if isinstance(v, int) else tuple(int(t) for t in v)


class _Pooling2D(Layer):
    _mode = 'max'

    def __init__(self, pool_size=(2, 2), strides=None, padding='valid', data_format=None, **kwargs):
        if data_format not in (None, 'channels_last'):
            raise NotImplementedError('pooling: channels_last only')
        super().__init__(**kwargs)
        self.pool_size = _pair(pool_size)
        self.strides = _pair(strides) if strides is not None else self.pool_size
        self.padding = padding.lower()
        if self.padding not in ('valid', 'same'):
            raise ValueError(f'unknown padding {padding!r}')

    def compute_output_shape(self, input_shape):
        out = [input_shape[0]]
        for n, p, s in zip(input_shape[1:3], self.pool_size, self.strides):
            out.append(None if n is None else (-(-n // s) if self.padding == 'same' else (n - p) // s + 1))
        return tuple(out) + (input_shape[3],)

    def call(self, x, training=None):
        return ops.pool2d(x, self.pool_size, self.strides, self.padding, self._mode)

    def get_config(self):
        return {'name': self.name, 'pool_size': self.pool_size, 'strides': self.strides, 'padding': self.padding}

    def host_fn(self, x):
        """The same pooling on a CPU tensor with library routines (for checks against a CPU model)."""
        import torch.nn.functional as F

        t = x.permute(0, 3, 1, 2)
        pads = [0, 0, 0, 0]
        if self.padding == 'same':
            pads = []
            for d in (1, 0):
                n, k, st = t.shape[2 + d], self.pool_size[d], self.strides[d]
                total = max((-(-n // st) - 1) * st + k - n, 0)
                pads += [total // 2, total - total // 2]
        if self._mode == 'max':
            y = F.max_pool2d(F.pad(t, pads, value=float('-inf')), self.pool_size, self.strides)
        else:
            num = F.avg_pool2d(F.pad(t, pads), self.pool_size, self.strides, divisor_override=1)
            cnt = F.avg_pool2d(F.pad(torch.ones_like(t[:1, :1]), pads), self.pool_size, self.strides, divisor_override=1)
            y = num / cnt
        return y.permute(0, 2, 3, 1)


class MaxPooling2D(_Pooling2D):
    _mode = 'max'


class AveragePooling2D(_Pooling2D):
    _mode = 'avg'


class Flatten(Layer):
    def compute_output_shape(self, input_shape):
        n = 1
        for d in input_shape[1:]:
            n *= d
        return (input_shape[0], n)

    def call(self, x, training=None):
        return x.reshape(x.shape[0], -1)

    host_fn = staticmethod(lambda x: x.reshape(x.shape[0], -1))


class GlobalAveragePooling1D(Layer):
    """Mean over the middle axis of a [batch, steps, channels] tensor."""

    def compute_output_shape(self, input_shape):
        return (input_shape[0], input_shape[2])

    def call(self, x, training=None):
        if x.is_cuda and x.dtype == torch.float32 and x.numel():
            return ops.mean_mid(x)
        return torch.mean(x, dim=1)

    host_fn = staticmethod(lambda x: torch.mean(x, dim=1))


layers = SimpleNamespace(MaxPooling2D=MaxPooling2D, AveragePooling2D=AveragePooling2D, Flatten=Flatten,
                         GlobalAveragePooling1D=GlobalAveragePooling1D, Layer=Layer)
