"""The generic quantizer layer (reference src/hgq/quantizer/quantizer.py:10-104): wraps an
internal quantizer and adds the optional scaler, quantization-noise blend and affine map."""

from __future__ import annotations

import torch

from ..core import Layer, base_name
from .config import QuantizerConfig, all_quantizer_keys


class Quantizer(Layer):
    """``Quantizer(config)`` or ``Quantizer(q_type=..., place=..., **quantizer_kwargs)``."""

    def __init__(self, *args, **kwargs):
        self.supports_masking = True
        config, kwargs = self.get_quantizer_config_kwargs(*args, **kwargs)
        super().__init__(**kwargs)
        self.config = config
        self.qnoise_factor = config.qnoise_factor
        self.scaler = config.scaler
        self.affine = config.affine
        self.quantizer = config.get_quantizer()
        # the one inner quantizer is named after its class alone: variable paths must not depend on how many
        # quantizers the process has created before
        self.quantizer.name = base_name(type(self.quantizer).__name__)

    def build(self, input_shape):
        if not self.quantizer.built:
            self.quantizer._build_device = self._build_device
            self.quantizer.build(tuple(input_shape))
            self.quantizer.built = True
        self.built = True

    def get_quantizer_config_kwargs(self, *args, **kwargs):
        if len(args) == 1 and isinstance(args[0], QuantizerConfig):
            return args[0], kwargs
        config = kwargs.pop('config', None)
        if isinstance(config, QuantizerConfig):
            return config, kwargs
        assert config is None, f'config must be a QuantizerConfig object, got {config}'
        q_kwargs = {k: kwargs.pop(k) for k in list(kwargs) if k in all_quantizer_keys}
        return QuantizerConfig(*args, **q_kwargs), kwargs

    def call(self, inputs, training=None):
        from .. import ops

        if self.scaler is not None:
            # a true division (on the GPU the tensor library divides by a Python number with a multiplication by its rounded
            # reciprocal, one ulp away from the quotient for some inputs - and one quantization step after rounding)
            inputs = ops.quantizer_scale_div(inputs, self.scaler)
        outputs = self.quantizer(inputs, training=training)
        # the multiplication by the scaler, the noise blend of training calls and the affine map: one pass each way
        return ops.quantizer_tail(outputs, inputs, self.scaler, self.qnoise_factor if training else None, self.affine)

    @property
    def plain(self) -> bool:
        """No scaler / noise blend / affine: the call is exactly the internal quantizer."""
        return self.scaler is None and self.qnoise_factor is None and self.affine is None

    def get_config(self):
        return {'name': self.name, 'config': self.config}

    @property
    def bits(self):
        return self.quantizer.bits

    @property
    def fbits(self):
        return self.quantizer.fbits

    @property
    def q_type(self):
        return self.config.q_type

    def __repr__(self):
        return f'{self.__class__.__name__}(q_type={self.config.q_type}, name={self.name}, built={self.built})'

    def bits_operand(self, shape):
        """``bits_(shape)`` as the operand of a fused EBOPs kernel (``ops.bits_ebops``): the raw variables and the
        broadcast rule ``(k, i, fb, size, inner, kbi, add_mode)``, or ``None`` when that form does not apply."""
        from .internal import FixedPointQuantizerKBI, FixedPointQuantizerKIF
        from .internal.base import bw_layout

        inner = self.quantizer
        if not isinstance(inner, (FixedPointQuantizerKIF, FixedPointQuantizerKBI)) or not inner.built:
            return None
        kbi = isinstance(inner, FixedPointQuantizerKBI)
        fb = inner._third()
        tensors = (inner._k, fb) if kbi else (inner._k, inner._i, fb)
        if not all(t.is_cuda and t.is_contiguous() for t in tensors) or fb.dtype != torch.float32:
            return None
        layout = bw_layout(fb.shape, tuple(shape))
        if layout is None:
            return None
        return (inner._k, None if kbi else inner._i, fb, layout[0], layout[1], kbi, 1 if inner.overflow_mode == 'SAT' else 0)

    def _bw_to_x(self, t, shape):
        t = torch.as_tensor(t)
        return self.quantizer.bw_mapper.bw_to_x(t, shape)

    def bits_(self, shape):
        return self._bw_to_x(self.bits, shape)

    def fbits_(self, shape):
        return self._bw_to_x(self.fbits, shape)

    def min_(self, shape):
        return self._bw_to_x(self.quantizer.min, shape)

    def max_(self, shape):
        return self._bw_to_x(self.quantizer.max, shape)

    def epsilon_(self, shape):
        return self._bw_to_x(self.quantizer.epsilon, shape)
