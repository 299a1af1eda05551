"""QEinsumDense (reference src/hgq/layers/core/einsum_dense.py:10-115).

Equations whose kernel axes are ``<contracted axes><new output axes>`` and whose input ends with
the contracted axes (``'bpf,fh->bph'``, ``'abc,cde->abde'``, ``'abcd,cde->abe'`` ...) reshape to
one GEMM and run through the fused dense kernels; every other equation quantizes the operands
with the quantizer kernels and contracts with ``torch.einsum``.
"""

from __future__ import annotations

import re
from math import prod

import torch

from ... import _lib, ops
from ...core import get_initializer
from ...quantizer import Quantizer
from ...quantizer.config import QuantizerConfig
from ._contraction import dense_contraction, dense_contraction_mean, dense_ebops_term, get_activation
from .base import QLayerBaseSingleInput, mean_bits, scale_ebops


def _einsum_free0_size(equation: str, input_shape) -> int:
    """Number of times the kernel is reused across the non-batch input axes."""
    _inp, _ker_out = equation.split(',', 1)
    _ker, _out = _ker_out.split('->', 1)
    elided_size = len(input_shape) - len(_inp) + 3
    _inp = _inp.replace('...', '?' * elided_size)
    n_parallel = 1
    for ax, dim in zip(_inp[1:], input_shape[1:]):
        if ax not in _ker and (ax in _out or ax == '?'):
            assert dim is not None, f'Cannot determine input loop size for einsum eq: {equation} with input shape {input_shape}'
            n_parallel *= dim
    return n_parallel


def analyze_einsum_string(equation, bias_axes, input_shape, output_shape):
    """Kernel shape, bias shape and full output shape of an EinsumDense equation (no ellipsis)."""
    m = re.match(r'([a-zA-Z]+),([a-zA-Z]+)->([a-zA-Z]+)', equation)
    if not m or '...' in equation:
        raise NotImplementedError(f'einsum equation {equation!r}: only ellipsis-free "ab,bc->ac" forms are supported')
    in_spec, w_spec, out_spec = m.groups()
    output_shape = [output_shape] if isinstance(output_shape, int) else list(output_shape)
    output_shape.insert(0, input_shape[0])
    if len(in_spec) != len(input_shape) or len(out_spec) != len(output_shape):
        raise ValueError(f'equation {equation} does not match input shape {input_shape} / output shape {output_shape}')
    in_map = {d: i for i, d in enumerate(in_spec)}
    out_map = {d: i for i, d in enumerate(out_spec)}
    for d in out_spec:
        if d not in in_spec and d not in w_spec:
            raise ValueError(f"Dimension '{d}' was specified in the output '{out_spec}' but has no corresponding dim")
    w_shape = []
    for d in w_spec:
        if d in in_map:
            w_shape.append(input_shape[in_map[d]])
        elif d in out_map:
            w_shape.append(output_shape[out_map[d]])
        else:
            raise ValueError(f"Weight dimension '{d}' did not have a match in either the input or the output spec")
    bias_shape = None
    if bias_axes is not None:
        for c in bias_axes:
            if c not in out_spec:
                raise ValueError(f"Bias dimension '{c}' was requested, but is not part of the output spec '{out_spec}'")
        first = min(out_spec.find(c) for c in bias_axes)
        bias_shape = [output_shape[out_map[c]] if c in bias_axes else 1 for c in out_spec[first:]]
    return tuple(w_shape), None if bias_shape is None else tuple(bias_shape), tuple(output_shape)


def gemm_form(equation):
    """(n_contract, n_new) if the equation is ``<free><C>,<C><O>-><free><O>``, else None."""
    in_spec, rest = equation.split(',', 1)
    w_spec, out_spec = rest.split('->', 1)
    for nc in range(1, len(w_spec)):
        c, o = w_spec[:nc], w_spec[nc:]
        if in_spec.endswith(c) and out_spec == in_spec[:len(in_spec) - nc] + o and not (set(o) & set(in_spec)):
            return nc, len(o)
    return None


def grouped_form(equation):
    """(n_group, n_contract, n_new) if the equation is ``<free><G><C>,<G><C><O>-><free><G><O>`` - the kernel carries the
    ``G`` axes of the input with it, one small kernel matrix per position (e.g. ``'Babc,bcd->Babd'``) - else None."""
    in_spec, rest = equation.split(',', 1)
    w_spec, out_spec = rest.split('->', 1)
    for ng in range(1, len(w_spec) - 1):
        for nc in range(1, len(w_spec) - ng):
            g, c, o = w_spec[:ng], w_spec[ng:ng + nc], w_spec[ng + nc:]
            if not o or not in_spec.endswith(g + c):
                continue
            free = in_spec[:len(in_spec) - ng - nc]
            if free and out_spec == free + g + o and not (set(o) & set(in_spec)) and len(set(w_spec)) == len(w_spec):
                return ng, nc, len(o)
    return None


class QEinsumDense(QLayerBaseSingleInput):
    def __init__(self, equation, output_shape, activation=None, bias_axes=None, kernel_initializer='glorot_uniform',
                 bias_initializer='zeros', kernel_regularizer=None, bias_regularizer=None, kernel_constraint=None,
                 bias_constraint=None, kq_conf: None | QuantizerConfig = None, iq_conf: None | QuantizerConfig = None,
                 bq_conf: None | QuantizerConfig = None, parallelization_factor: int = -1, **kwargs):
        super().__init__(iq_conf=iq_conf, **kwargs)
        self.equation = equation
        self.partial_output_shape = (output_shape,) if isinstance(output_shape, int) else tuple(output_shape)
        self.bias_axes = bias_axes
        self.activation, self._act_name = get_activation(activation)
        self.kernel_initializer = get_initializer(kernel_initializer)
        self.bias_initializer = get_initializer(bias_initializer)
        self.kernel_regularizer, self.bias_regularizer = kernel_regularizer, bias_regularizer
        self.kernel_constraint, self.bias_constraint = kernel_constraint, bias_constraint
        kq_conf = kq_conf or QuantizerConfig('default', 'weight')
        self._kq = Quantizer(kq_conf, name=f'{self.name}_kq')
        bq_conf = bq_conf or QuantizerConfig('default', 'bias')
        self._bq = None if bias_axes is None else Quantizer(bq_conf, name=f'{self.name}_bq')
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
        kernel_shape, bias_shape, full_output_shape = analyze_einsum_string(
            self.equation, self.bias_axes, tuple(input_shape), self.partial_output_shape)
        self.full_output_shape = tuple(full_output_shape)
        self._kernel = self.add_weight(name='kernel', shape=kernel_shape, initializer=self.kernel_initializer,
                                       regularizer=self.kernel_regularizer, constraint=self.kernel_constraint)
        if bias_shape is not None:
            self.bias = self.add_weight(name='bias', shape=bias_shape, initializer=self.bias_initializer,
                                        regularizer=self.bias_regularizer, constraint=self.bias_constraint)
        self.n_parallel = _einsum_free0_size(self.equation, input_shape)
        if self.parallelization_factor < 0:
            self.parallelization_factor = self.n_parallel
        for q, shape in ((self.kq, kernel_shape), (self.bq, bias_shape)):
            if q is not None:
                q._build_device = self._build_device
                q.build(tuple(shape))
                q.built = True
        self.ebops_equation = self.equation.split('->')[0] + '->'
        self._gemm = gemm_form(self.equation)
        self._grouped = grouped_form(self.equation) if self._gemm is None else None
        if self._grouped is not None:
            ng, nc, _ = self._grouped
            self._G, self._gK, self._gN = prod(kernel_shape[:ng]), prod(kernel_shape[ng:ng + nc]), prod(kernel_shape[ng + nc:])
            # the bias rides in the kernel only when it is exactly one value per (group, output column)
            self._bias_in_grouped = bias_shape is not None and prod(bias_shape) == self._G * self._gN and \
                tuple(s for s in bias_shape if s != 1) == tuple(s for s in kernel_shape[:ng] + kernel_shape[ng + nc:] if s != 1)
        if self._gemm is not None:
            nc, _ = self._gemm
            self._K = prod(kernel_shape[:nc])
            self._N = prod(kernel_shape[nc:])
            # the bias rides in the GEMM epilogue only when it is exactly one value per output column
            self._bias_in_gemm = bias_shape is not None and prod(bias_shape) == self._N and \
                tuple(s for s in bias_shape if s != 1) == tuple(s for s in kernel_shape[nc:] if s != 1)
        if self.enable_oq and not self.oq.built:
            # the output shape is known only now (the reference's parent class sets it before the base class builds the
            # output quantizer, src/hgq/layers/core/base.py:183-186)
            self.try_build_output_quantizer(input_shape)

    def compute_output_shape(self, input_shape):
        return (input_shape[0],) + tuple(self.full_output_shape[1:])

    def absorbs(self, nxt, x) -> bool:
        """Whether a call may take the layer that follows in a :class:`Sequential` with it (``call(..., then=nxt)``): a mean
        over the middle axis of a [batch, positions, channels] output (32 or 64 positions) behind a linear or ReLU contraction
        over the trailing input axis, without output quantizer.  The contraction kernel then writes the means as its tiles leave,
        and the backward pass reads the means' gradient instead of a broadcast copy."""
        from ...host import GlobalAveragePooling1D

        if type(nxt) is not GlobalAveragePooling1D or not getattr(type(self).call, '_takes_then', False) or not self.built:
            return False
        if self.enable_oq or self._act_name not in (None, 'linear', 'relu') or not torch.is_tensor(x) or not x.is_cuda or x.dim() != 3:
            return False
        out = tuple(self.full_output_shape)
        return (self._gemm is not None and len(out) == 3 and out[-1] == self._N and x.shape[-1] == self._K and out[1] == x.shape[1]
                and x.shape[1] in (32, 64) and (self.bias is None or self._bias_in_gemm))

    def _contract(self, inputs, qkernel, qbias, training, oq_ok=False, mean_rows=0):
        """``(outputs, activation applied)``; with ``mean_rows`` (a call that absorbed the mean over the middle axis)
        ``(outputs, activation applied, mean taken)``."""
        if mean_rows:
            y, act_done, mean_done = self._contract_mean(inputs, qkernel, qbias, training, mean_rows)
            if mean_done:
                return y, act_done, True
            return self._contract(inputs, qkernel, qbias, training, oq_ok) + (False,)
        iq = self.iq if self.enable_iq else None
        if self._gemm is not None:
            nc, _ = self._gemm
            x = inputs  # the contracted axes are trailing and contiguous: a [rows, K] view of the same memory
            b1d = qbias.reshape(-1) if (qbias is not None and self._bias_in_gemm) else None
            fuse_act = self._act_name if (qbias is None or self._bias_in_gemm) else None
            w2d = qkernel.reshape(self._K, self._N)
            # a view's gradient goes back through the view unread: the "one reader" mark of a prefetched operand holds for it
            for view, base in ((w2d, qkernel), (b1d, qbias)):
                if (view is not None and view is not base and getattr(base, '_hgq_single_use', False)
                        and view._base is not None and view.data_ptr() == base.data_ptr() and view.numel() == base.numel()):
                    view._hgq_single_use = True  # the same elements under another shape
            # the output quantizer can join the kernel when nothing but the fused activation follows the contraction
            oq = None
            if oq_ok and self.enable_oq and not self.__output_quantizer_handled__ and (qbias is None or self._bias_in_gemm):
                oq = self.oq
            y, act_done, self._deferred, oq_done = dense_contraction(x, iq, w2d, b1d, fuse_act, training, oq,
                                                                     (inputs.shape[0],) + tuple(self.full_output_shape[1:]))
            if oq_done:
                self._oq_applied_in_call = True
            y = y.view(inputs.shape[0], *self.full_output_shape[1:])
            if qbias is not None and not self._bias_in_gemm:
                y = ops.bias_add_rows(y, qbias)
            return y, act_done
        if iq is not None:
            inputs = iq(inputs, training=training)
        if self._grouped is not None and inputs.is_cuda and inputs.numel() > 0:
            # one small kernel matrix per position: the grouped dense kernels on [rows, G, K] / [G, K, N] views
            x3 = inputs.reshape(-1, self._G, self._gK)
            w3 = qkernel.reshape(self._G, self._gK, self._gN)
            if ops.gdense_supported(x3, w3):
                in_kernel = qbias is None or self._bias_in_grouped
                relu = in_kernel and self._act_name == 'relu'
                y = ops.gdense(x3, w3, qbias.reshape(self._G, self._gN) if (qbias is not None and in_kernel) else None,
                               _lib.ACT_RELU if relu else _lib.ACT_NONE)
                y = y.view(inputs.shape[0], *self.full_output_shape[1:])
                if qbias is not None and not in_kernel:
                    y = ops.bias_add_rows(y, qbias)
                return y, relu or (in_kernel and self._act_name == 'linear')
        y = torch.einsum(self.equation, inputs, qkernel)
        if qbias is not None:
            y = ops.bias_add_rows(y, qbias)
        return y, False

    def _contract_mean(self, inputs, qkernel, qbias, training, mean_rows):
        """The contraction and the mean over the middle axis in one launch each way where the kernels cover it:
        ``(means, True, True)``, else ``(None, False, False)``."""
        if self._gemm is None or (qbias is not None and not self._bias_in_gemm):
            return None, False, False
        w2d = qkernel.reshape(self._K, self._N)
        b1d = qbias.reshape(-1) if qbias is not None else None
        for view, base in ((w2d, qkernel), (b1d, qbias)):
            if (view is not None and view is not base and getattr(base, '_hgq_single_use', False)
                    and view._base is not None and view.data_ptr() == base.data_ptr() and view.numel() == base.numel()):
                view._hgq_single_use = True  # the same elements under another shape
        r = dense_contraction_mean(inputs, self.iq if self.enable_iq else None, w2d, b1d, self._act_name, training, mean_rows)
        if r is None:
            return None, False, False
        y, self._deferred = r
        return y, True, True

    def _finish_then(self, y, act_done, mean_done, then):
        """The tail of a call that absorbed the layer behind it: whatever the kernels did not take."""
        if self.activation is not None and not act_done:
            y = self.activation(y)
        return y if mean_done else then(y)

    def call(self, inputs, training=None, then=None):
        qkernel = self.kq(self._kernel, training=training)
        qbias = self.bq(self.bias, training=training) if self.bias is not None else None
        if then is not None:
            return self._finish_then(*self._contract(inputs, qkernel, qbias, training, mean_rows=inputs.shape[1]), then)
        y, act_done = self._contract(inputs, qkernel, qbias, training, oq_ok=True)
        if self.activation is not None and not act_done:
            y = self.activation(y)
        return y

    call._takes_then = True

    def _finish_call(self):
        d, self._deferred = getattr(self, '_deferred', None), None
        if d is not None:
            d.flush()

    def _ebops_loss_term(self, shape):
        out_size = float(prod(self.full_output_shape[1:]))
        if self._gemm is not None and (self.bq is None or self._bias_in_gemm):
            term = dense_ebops_term(self, self.iq, self.kq, self.bq, self._K, self._N, out_size,
                                    getattr(self, '_deferred', None))
            if term is not None:
                return term
        self._finish_call()
        return super()._ebops_loss_term(shape)

    def _compute_ebops(self, shape):
        out_size = float(prod(self.full_output_shape[1:]))
        bw_inp = self.iq.bits_(shape)
        bw_ker = self.kq.bits_(self._kernel.shape)
        ebops = torch.einsum(self.ebops_equation, bw_inp, bw_ker)
        if self.bq is not None:
            bw_bias = self.bq.bits_(self.bias.shape)
            ebops = ebops + mean_bits(bw_bias) * out_size
        return scale_ebops(ebops, self.parallelization_factor, self.n_parallel)

    def get_config(self):
        config = super().get_config()
        config.update({'equation': self.equation, 'output_shape': self.partial_output_shape, 'bias_axes': self.bias_axes,
                       'activation': self._act_name, 'kq_conf': self.kq.config,
                       'bq_conf': self.bq.config if self.bq is not None else None,
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
