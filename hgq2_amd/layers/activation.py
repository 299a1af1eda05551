"""QUnaryFunctionLUT (reference src/hgq/layers/activation.py:18-67): ``oq(f(iq(x)))``, i.e. a
function that will be realised as a lookup table; EBOPs ``sum(2**bits_in * bits_out) * 1e-4``."""

from __future__ import annotations

from collections.abc import Callable

import torch

from ..quantizer import QuantizerConfig
from .core._contraction import get_activation
from .core.base import QLayerBaseSingleInput


class QUnaryFunctionLUT(QLayerBaseSingleInput):
    def __init__(self, activation: Callable | str, iq_conf: QuantizerConfig | None = None,
                 oq_conf: QuantizerConfig | None = None, enable_oq=True, enable_iq=True,
                 allow_heterogeneous_input: bool = True, allow_heterogeneous_table: bool = True,
                 override_oq_k0_to_0: bool = False, **kwargs):
        act_name = activation.__name__ if isinstance(activation, Callable) else activation
        assert act_name not in ('softmax', 'log_softmax'), f'activation {act_name} is not unary'
        self._allow_heterogeneous_table = allow_heterogeneous_table
        self._allow_heterogeneous_input = allow_heterogeneous_input
        disable_ebops = False
        if enable_oq:
            oq_conf = oq_conf or QuantizerConfig('default', 'table')
            if override_oq_k0_to_0 and 'k0' in oq_conf.config:
                oq_conf.config['k0'] = False
            if not allow_heterogeneous_table:
                oq_conf.config['homogeneous_axis'] = None
                oq_conf.config['heterogeneous_axis'] = ()
        else:
            disable_ebops = True
        if enable_iq and not allow_heterogeneous_input:
            iq_conf = iq_conf or QuantizerConfig('default', 'datalane')
            iq_conf.config['homogeneous_axis'] = None
            iq_conf.config['heterogeneous_axis'] = ()
        super().__init__(iq_conf=iq_conf, oq_conf=oq_conf, enable_oq=enable_oq, enable_iq=enable_iq, **kwargs)
        if disable_ebops:
            self._enable_ebops = False
        self.activation, self._act_name = get_activation(activation)
        if self.activation is None:
            self.activation = lambda x: x

    def call(self, inputs, training=None):
        if self.enable_iq:
            inputs = self.iq(inputs, training=training)
        return self.activation(inputs)

    def _ebops_loss_term(self, shape):
        # value, uint32 variable, loss term and the bit-width gradients in one launch where the quantizers allow it
        if self.enable_iq and self.enable_oq and self._beta is not None and self._beta.is_cuda:
            operands = [self.iq.bits_operand(shape), self.oq.bits_operand(shape)]
            n_cells = 1
            for s in shape:
                n_cells *= int(s)
            if all(op is not None for op in operands) and 0 < n_cells < 2**31 and sum(op[3] for op in operands) <= 30720:
                from .. import ops

                return ops.bits_ebops('lut', operands, (n_cells, 1e-4, float(self.ebops_factor)), self._beta, self._ebops)
        return super()._ebops_loss_term(shape)

    def _compute_ebops(self, shape):
        bw_inp = self.iq.bits_(shape)
        bw_out = self.oq.bits_(shape)
        return torch.sum((2.0**bw_inp) * bw_out) * 1e-4

    def get_config(self):
        config = super().get_config()
        config['activation'] = self._act_name  # a named activation; a callable has to be passed again on loading
        config['allow_heterogeneous_table'] = self._allow_heterogeneous_table
        config['allow_heterogeneous_input'] = self._allow_heterogeneous_input
        return config
