"""QConv2D (reference src/hgq/layers/conv.py:12-102,175-200): ``act(conv(iq(x), kq(W)) + bq(b))``
on channels-last tensors with the kernel in HWIO layout, and the EBOPs obtained by convolving the
bit-width tensors.  The input / kernel / bias quantizers run in the HIP quantizer kernels; the
convolution of the quantized operands, the bias add and a ReLU run in the implicit-GEMM kernels
(``hgq_conv2d_fwd / hgq_conv2d_bwd``), which are also what convolves the bit-width tensors for EBOPs."""

from __future__ import annotations

from math import prod

import torch

from .. import _lib, ops

from ..core import get_initializer
from ..quantizer import Quantizer
from ..quantizer.config import QuantizerConfig
from .core._contraction import get_activation
from .core.base import QLayerBaseSingleInput, mean_bits


def _pair(v):
    return (int(v), int(v)) if isinstance(v, int) else tuple(int(t) for t in v)


class QConv2D(QLayerBaseSingleInput):
    def __init__(self, filters, kernel_size, strides=(1, 1), padding='valid', data_format=None, dilation_rate=(1, 1),
                 groups=1, activation=None, use_bias=True, kernel_initializer='glorot_uniform', bias_initializer='zeros',
                 kernel_regularizer=None, bias_regularizer=None, activity_regularizer=None, kernel_constraint=None,
                 bias_constraint=None, kq_conf: None | QuantizerConfig = None, iq_conf: None | QuantizerConfig = None,
                 bq_conf: None | QuantizerConfig = None, parallelization_factor=-1, **kwargs):
        super().__init__(iq_conf=iq_conf, **kwargs)
        if data_format not in (None, 'channels_last'):
            raise NotImplementedError('QConv2D: channels_last only')
        if groups != 1:
            raise NotImplementedError('QConv2D: groups == 1 only')
        self.rank = 2
        self.filters = int(filters)
        self.kernel_size, self.strides, self.dilation_rate = _pair(kernel_size), _pair(strides), _pair(dilation_rate)
        self.padding = padding.lower()
        assert self.padding in ('valid', 'same')
        self.data_format = 'channels_last'
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

    def compute_output_shape(self, input_shape):
        out = [input_shape[0]]
        for d, (k, s, dil) in enumerate(zip(self.kernel_size, self.strides, self.dilation_rate)):
            n = input_shape[1 + d]
            if n is None:
                out.append(None)
            elif self.padding == 'same':
                out.append(-(-n // s))
            else:
                out.append((n - dil * (k - 1) - 1) // s + 1)
        return tuple(out) + (self.filters,)

    def build(self, input_shape):
        super().build(input_shape)
        c_in = int(input_shape[-1])
        self._kernel = self.add_weight(name='kernel', shape=self.kernel_size + (c_in, self.filters),
                                       initializer=self.kernel_initializer, regularizer=self.kernel_regularizer,
                                       constraint=self.kernel_constraint)
        if self.use_bias:
            self.bias = self.add_weight(name='bias', shape=(self.filters,), initializer=self.bias_initializer,
                                        regularizer=self.bias_regularizer, constraint=self.bias_constraint)
        for q, shape in ((self.kq, self._kernel.shape), (self.bq, (self.filters,))):
            if q is not None:
                q._build_device = self._build_device
                q.build(tuple(shape))
                q.built = True
        out_shape = self.compute_output_shape(input_shape)
        self.n_parallel = None if None in out_shape[1:] else prod(out_shape[1:-1])
        if self.parallelization_factor <= 0:
            assert self.n_parallel is not None
            self.parallelization_factor = self.n_parallel

    def convolution_op(self, x_nhwc, kernel_hwio, bias=None, act_code=_lib.ACT_NONE, maxpool2=False):
        """``act(conv(x, kernel) + bias)`` on channels-last tensors through the implicit-GEMM kernels."""
        return ops.conv2d(x_nhwc, kernel_hwio, bias, self.strides, self.padding, self.dilation_rate, act_code, maxpool2)

    def absorbs(self, nxt, x) -> bool:
        """Whether a call may take the layer that follows in a :class:`Sequential` with it (``call(..., then=nxt)``): a plain
        2 x 2 maximum pooling of stride 2 behind a linear or ReLU convolution without output quantizer, on a shape the
        kernels take.  The unpooled output then never leaves the layer, and its backward pass starts from the pooled gradient."""
        from ..host import MaxPooling2D

        if type(nxt) is not MaxPooling2D or nxt.pool_size != (2, 2) or nxt.strides != (2, 2) or nxt.padding != 'valid':
            return False
        if type(self).call is not QConv2D.call or type(self).convolution_op is not QConv2D.convolution_op:
            return False  # a subclass with its own call: it does not know the `then` argument
        if self.enable_oq or self._act_name not in (None, 'linear', 'relu') or not torch.is_tensor(x) or not x.is_cuda or x.dim() != 4:
            return False
        geom = ops.conv_geometry(tuple(x.shape), self.kernel_size + (x.shape[-1], self.filters), self.strides, self.padding, self.dilation_rate)
        return geom[0] > 0 and ops.conv2d_maxpool_supported(geom, self.filters)

    def call(self, inputs, training=None, then=None):
        if self.enable_iq:
            inputs = self.iq(inputs, training=training)
        fused_act = _lib.ACT_RELU if self._act_name == 'relu' else _lib.ACT_NONE
        if then is not None:
            return self.convolution_op(inputs, self.qkernel, self.qbias if self.use_bias else None, fused_act, True)
        outputs = self.convolution_op(inputs, self.qkernel, self.qbias if self.use_bias else None, fused_act)
        if self.activation is not None and fused_act == _lib.ACT_NONE:
            outputs = self.activation(outputs)
        return outputs

    def _ebops_loss_term(self, shape):
        # the whole estimate, the uint32 variable, the loss term and the bit-width gradients in one launch where every
        # quantizer has one bit-width entry per cell
        if self.enable_iq and self._beta is not None and self._beta.is_cuda:
            operands = [self.iq.bits_operand(shape), self.kq.bits_operand(tuple(self._kernel.shape)),
                        self.bq.bits_operand((self.filters,)) if self.bq is not None else None]
            cells = [prod(shape), self._kernel.numel(), self.filters]
            ok = all(op is None or (op[3] == n and op[4] == 1) for op, n in zip(operands, cells)) and operands[0] is not None \
                and operands[1] is not None and (self.bq is None or operands[2] is not None)
            if ok and ops.conv2d_ebops_supported(tuple(shape), tuple(self._kernel.shape)):
                geom = ops.conv_geometry(tuple(shape), tuple(self._kernel.shape), self.strides, self.padding, self.dilation_rate)
                size = float(prod(shape[:-1]) * self.filters)
                return ops.bits_ebops('conv', operands, (tuple(geom), self.filters, self.parallelization_factor / self.n_parallel, size,
                                                         float(self.ebops_factor)), self._beta, self._ebops)
        return super()._ebops_loss_term(shape)

    def _compute_ebops(self, shape):
        bw_inp = self.iq.bits_(shape)
        bw_ker = self.kq.bits_(self._kernel.shape)
        if bw_inp.is_cuda and ops.conv2d_ebops_supported(tuple(bw_inp.shape), tuple(bw_ker.shape)):
            ebops = ops.conv2d_ebops(bw_inp, bw_ker, self.strides, self.padding, self.dilation_rate)
        else:
            ebops = torch.sum(self.convolution_op(bw_inp, bw_ker))
        ebops = ebops * (self.parallelization_factor / self.n_parallel)
        if self.bq is not None:
            size = float(prod(shape[:-1]) * self.filters)
            bw_bias = self.bq.bits_(self.bias.shape)
            ebops = ebops + mean_bits(bw_bias) * size
        return ebops

    def get_config(self):
        config = super().get_config()
        config.update({'filters': self.filters, 'kernel_size': self.kernel_size, 'strides': self.strides, 'padding': self.padding,
                       'dilation_rate': self.dilation_rate, 'activation': self._act_name, 'use_bias': self.use_bias,
                       'kernel_initializer': self.kernel_initializer, 'bias_initializer': self.bias_initializer,
                       'kq_conf': self.kq.config, 'bq_conf': self.bq.config if self.bq is not None else None,
                       'parallelization_factor': self.parallelization_factor})
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
