"""QDense (reference src/hgq/layers/core/dense.py:12-102)."""

from __future__ import annotations

from math import prod

import torch

from ...core import get_initializer
from ...quantizer import Quantizer
from ...quantizer.config import QuantizerConfig
from ._contraction import dense_contraction, dense_ebops_term, get_activation
from .base import QLayerBaseSingleInput, mean_bits, scale_ebops


class QDense(QLayerBaseSingleInput):
    """``activation(iq(x) @ kq(kernel) + bq(bias))`` with per-weight / per-activation bit-widths."""

    def __init__(self, units, activation=None, use_bias=True, kernel_initializer='glorot_uniform',
                 bias_initializer='zeros', kernel_regularizer=None, bias_regularizer=None, activity_regularizer=None,
                 kernel_constraint=None, bias_constraint=None, kq_conf: None | QuantizerConfig = None,
                 iq_conf: None | QuantizerConfig = None, bq_conf: None | QuantizerConfig = None,
                 parallelization_factor=-1, **kwargs):
        super().__init__(iq_conf=iq_conf, **kwargs)
        self.units = int(units)
        self.activation, self._act_name = get_activation(activation)
        self.use_bias = use_bias
        self.kernel_initializer = get_initializer(kernel_initializer)
        self.bias_initializer = get_initializer(bias_initializer)
        self.kernel_regularizer, self.bias_regularizer = kernel_regularizer, bias_regularizer
        self.kernel_constraint, self.bias_constraint = kernel_constraint, bias_constraint
        kq_conf = kq_conf or QuantizerConfig('default', 'weight')
        self._kq = Quantizer(kq_conf, name=f'{self.name}_kq')
        bq_conf = bq_conf or QuantizerConfig('default', 'bias')
        self._bq = Quantizer(bq_conf, name=f'{self.name}_bq') if use_bias else None
        self.parallelization_factor = parallelization_factor
        self.bias = None

    @property
    def kq(self):
        return self._kq

    @property
    def bq(self):
        return self._bq

    @property
    def kernel(self):
        return self._kernel

    def build(self, input_shape):
        super().build(input_shape)
        k_in = int(input_shape[-1])
        self._kernel = self.add_weight(name='kernel', shape=(k_in, self.units), initializer=self.kernel_initializer,
                                       regularizer=self.kernel_regularizer, constraint=self.kernel_constraint)
        if self.use_bias:
            self.bias = self.add_weight(name='bias', shape=(self.units,), initializer=self.bias_initializer,
                                        regularizer=self.bias_regularizer, constraint=self.bias_constraint)
        self.n_parallel = prod(input_shape[1:-1])
        if self.parallelization_factor < 0:
            self.parallelization_factor = self.n_parallel
        for q, shape in ((self.kq, self._kernel.shape), (self.bq, (self.units,))):
            if q is not None:
                q._build_device = self._build_device
                q.build(tuple(shape))
                q.built = True

    def compute_output_shape(self, input_shape):
        return tuple(input_shape[:-1]) + (self.units,)

    def call(self, inputs, training=None):
        iq = self.iq if self.enable_iq else None
        oq = self.oq if (self.enable_oq and not self.__output_quantizer_handled__) else None
        y, act_done, self._deferred, self._oq_applied_in_call = dense_contraction(
            inputs, iq, self.qkernel, self.qbias, self._act_name, training, oq, tuple(inputs.shape[:-1]) + (self.units,))
        y = y.view(*inputs.shape[:-1], self.units)
        if self.activation is not None and not act_done:
            y = self.activation(y)
        return y

    def _finish_call(self):
        d, self._deferred = getattr(self, '_deferred', None), None
        if d is not None:
            d.flush()

    def _ebops_loss_term(self, shape):
        out_size = float(prod(shape[:-1]) * self.units)
        term = dense_ebops_term(self, self.iq, self.kq, self.bq, shape[-1], self.units, out_size,
                                getattr(self, '_deferred', None))
        if term is not None:
            return term
        self._finish_call()  # the generic path reads the integer bits: track first
        return super()._ebops_loss_term(shape)

    def _compute_ebops(self, shape):
        out_size = float(prod(shape[:-1]) * self.units)
        bw_inp = self.iq.bits_(shape)
        bw_ker = self.kq.bits_(self._kernel.shape).to(bw_inp.device)
        ebops = torch.sum(torch.matmul(bw_inp, bw_ker))
        if self.bq is not None:
            bw_bias = self.bq.bits_(self.bias.shape)
            ebops = ebops + mean_bits(bw_bias) * out_size
        return scale_ebops(ebops, self.parallelization_factor, self.n_parallel)

    def get_config(self):
        config = super().get_config()
        config.update({'units': self.units, 'activation': self._act_name, 'use_bias': self.use_bias,
                       'kq_conf': self.kq.config, 'bq_conf': self.bq.config if self.bq is not None else None,
                       'parallelization_factor': self.parallelization_factor,
                       'kernel_initializer': self.kernel_initializer, 'bias_initializer': self.bias_initializer})
        return config

    def _weight_quantizer_inputs(self):
        """(quantizer, variable) pairs this layer's call quantizes as they are: candidates for the batched launch
        ahead of the forward pass (quantizer/prefetch.py)."""
        pairs = [(self.kq, self._kernel)]
        if self.bias is not None and self.bq is not None:
            pairs.append((self.bq, self.bias))
        return pairs

    @property
    def qkernel(self):
        return self.kq(self._kernel)

    @property
    def qbias(self):
        if self.bias is None:
            return None
        return self.bq(self.bias)
