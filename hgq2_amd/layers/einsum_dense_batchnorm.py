"""QEinsumDenseBatchnorm (reference src/hgq/layers/einsum_dense_batchnorm.py:11-211): batch
normalisation folded into the kernel and bias *before* they are quantized.  In training the
moments come from an un-quantized-kernel contraction of the quantized input, so each step runs
two contractions."""

from __future__ import annotations

import numpy as np
import torch

from .. import _lib, ops
from ..core import epsilon, get_initializer
from ..quantizer.prefetch import _eligible, quantize_together
from .core._contraction import fused_iq_rows
from .core.einsum_dense import QEinsumDense, analyze_einsum_string


class QEinsumDenseBatchnorm(QEinsumDense):
    def __init__(self, equation, output_shape, activation=None, bias_axes=None, normalize_axes: str | None = None,
                 momentum=0.99, epsilon=1e-3, center=True, scale=True, beta_initializer='zeros',
                 gamma_initializer='ones', moving_mean_initializer='zeros', moving_variance_initializer='ones',
                 beta_regularizer=None, gamma_regularizer=None, beta_constraint=None, gamma_constraint=None,
                 synchronized=False, **kwargs):
        super().__init__(equation=equation, output_shape=output_shape, activation=activation, bias_axes=bias_axes, **kwargs)
        self.synchronized = synchronized
        self.momentum = float(momentum)
        self.epsilon = float(epsilon)  # stored only: the fusion uses the global epsilon, as the reference does (:165)
        self.center = center
        self.scale = scale
        self.gamma_initializer = get_initializer(gamma_initializer)
        self.moving_mean_initializer = get_initializer(moving_mean_initializer)
        self.moving_variance_initializer = get_initializer(moving_variance_initializer)
        self.gamma_regularizer, self.gamma_constraint = gamma_regularizer, gamma_constraint
        normalize_axes = normalize_axes or bias_axes
        assert normalize_axes is not None, 'Either normalize_axes or bias_axes must be provided.'
        self.normalize_axes = normalize_axes
        self._check_normalize_axes()

    def get_config(self):
        config = super().get_config()
        config.update({'normalize_axes': self.normalize_axes, 'momentum': self.momentum, 'epsilon': self.epsilon, 'center': self.center,
                       'scale': self.scale, 'gamma_initializer': self.gamma_initializer,
                       'moving_mean_initializer': self.moving_mean_initializer,
                       'moving_variance_initializer': self.moving_variance_initializer, 'synchronized': self.synchronized})
        return config

    def _check_normalize_axes(self):
        kernel_axes, output_axes = self.equation.split(',')[1].split('->')
        for c in self.normalize_axes:
            if c not in kernel_axes:
                raise ValueError(f'Axis {c} not found in kernel axes {kernel_axes}')
            if c not in output_axes:
                raise ValueError(f'Axis {c} not found in output axes {output_axes}')
            if self.bias_axes and c not in self.bias_axes:
                raise ValueError(f'Axis {c} not found in bias axes {self.bias_axes}')

    def _compute_fused_einsum_specs(self, input_shape):
        kernel_axes, output_axes = self.equation.split(',')[1].split('->')
        _, norm_cast_shape, output_shape = analyze_einsum_string(self.equation, self.normalize_axes, tuple(input_shape),
                                                                 self.partial_output_shape)
        normalize_axes = ''.join(c for c in kernel_axes if c in self.normalize_axes)
        self._reduction_axes = tuple(i for i, c in enumerate(output_axes) if c not in normalize_axes)
        norm_shape = tuple(output_shape[i] for i, c in enumerate(output_axes) if c in normalize_axes)
        assert np.prod(norm_shape) == np.prod(norm_cast_shape), f'{norm_shape} != {norm_cast_shape}'
        self._norm_offset_cast_shape = norm_cast_shape
        self.fused_kernel_equation = f'{kernel_axes},{normalize_axes}->{kernel_axes}'
        return norm_shape

    def build(self, input_shape):
        super().build(input_shape)
        norm_shape = self._compute_fused_einsum_specs(input_shape)
        if self.scale:
            self.bn_gamma = self.add_weight(shape=norm_shape, name='gamma', initializer=self.gamma_initializer,
                                            regularizer=self.gamma_regularizer, constraint=self.gamma_constraint)
        assert self.bias is not None
        self.bias.requires_grad_(bool(self.center))
        self.moving_mean = self.add_weight(shape=norm_shape, name='moving_mean', initializer=self.moving_mean_initializer,
                                           trainable=False)
        self.moving_variance = self.add_weight(shape=norm_shape, name='moving_variance',
                                               initializer=self.moving_variance_initializer, trainable=False)

    def get_fused_qkernel_and_qbias(self, training, mean, var):
        bn_gamma = self.bn_gamma if self.scale else 1
        scaler = bn_gamma / torch.sqrt(var + epsilon())
        fused_kernel = torch.einsum(self.fused_kernel_equation, self._kernel, scaler)
        fused_qkernel = self.kq(fused_kernel, training=training)
        offset = torch.reshape(-mean * scaler, self._norm_offset_cast_shape)
        fused_qbias = self.bq(self.bias + offset, training=training)
        return fused_qkernel, fused_qbias

    @property
    def qkernel(self):
        return self.get_fused_qkernel_and_qbias(False, self.moving_mean, self.moving_variance)[0]

    @property
    def qbias(self):
        return self.get_fused_qkernel_and_qbias(False, self.moving_mean, self.moving_variance)[1]

    def _weight_quantizer_inputs(self):
        return []  # kernel and bias are quantized after folding the batch statistics in: they depend on the input

    def _trailing_gemm(self):
        """GEMM-shaped equation whose normalised axes are exactly the new output axes."""
        n_out = len(self.full_output_shape)
        return self._gemm is not None and self._reduction_axes == tuple(range(n_out - self._gemm[1]))

    def _batch_moments(self, qinputs, raw=False, quant=None, chain=False):
        """Mean and variance (``raw``: mean of squares, flat) of the un-quantized-kernel pre-activation
        over the non-normalised axes (reference :108-112).  GEMM-shaped equations whose normalised axes
        are all the new output axes run through the dense and column-moment kernels; others through the
        library einsum.  ``chain`` (with ``raw``): a third result, the input to hand to the output contraction
        - the same values, routed so that its gradient is added inside the statistics' backward kernel -
        or ``None`` where the path taken has no such kernel."""
        n_out = len(self.full_output_shape)
        trailing = self._trailing_gemm()
        if trailing and qinputs.is_cuda:
            x2d = qinputs.reshape(-1, self._K)
            w2d = self._kernel.reshape(self._K, self._N)
            x2d = x2d.contiguous()
            alias = None
            if ops.dense_moments_supported(x2d, w2d):
                # one pass over x, the pre-activation is never written
                if chain and raw:
                    mean, meansq, alias = ops.dense_moments(x2d, w2d, quant, chain=True)
                    alias = alias.view(qinputs.shape)
                else:
                    mean, meansq = ops.dense_moments(x2d, w2d, quant)
            else:
                if self._K <= ops.FUSED_BWD_MAX and self._N <= ops.FUSED_BWD_MAX:
                    pre, _ = ops.qdense(x2d, None, None, None, w2d, None, _lib.ACT_NONE, 0, 0, False)
                else:
                    pre = ops.matmul_bias_act(x2d, w2d, None, _lib.ACT_NONE)
                mean, meansq = ops.col_moments(pre)
            if raw:
                return (mean, meansq, alias) if chain else (mean, meansq)
            shape = tuple(self.full_output_shape[n_out - self._gemm[1]:])
            mean, meansq = mean.view(shape), meansq.view(shape)
            return mean, meansq - torch.square(mean)
        x = torch.einsum(self.equation, qinputs, self._kernel)
        mean = torch.mean(x, dim=self._reduction_axes)
        return mean, torch.mean(torch.square(x), dim=self._reduction_axes) - torch.square(mean)

    def _fused_iq(self, inputs, training):
        """``(f_in, bw_rows, mode)`` if the input quantizer can run inside both contractions (statistics and output) while
        they stage their operand - the quantized input is then never written - else ``None``."""
        if not (self.enable_iq and training is True and self.trainable and inputs.is_cuda and self._trailing_gemm()):
            return None
        if self.bias.numel() != self._N or self._K > ops.FUSED_BWD_MAX or self._N > ops.FUSED_BWD_MAX:
            return None
        bw_rows = fused_iq_rows(self.iq, tuple(inputs.shape), self._K, training)
        x2d = inputs.reshape(-1, self._K)
        if not bw_rows or 64 % bw_rows or not x2d.is_contiguous() or not ops.dense_moments_supported(x2d, self._kernel.reshape(self._K, self._N)):
            return None
        q = self.iq.quantizer
        return q._f.view(-1), bw_rows, q._mode(True)

    def call(self, inputs, training=None, then=None):
        quant = self._fused_iq(inputs, training)
        if quant is None and self.enable_iq:
            inputs = self.iq(inputs, training=training)
        if training and self.trainable and inputs.is_cuda and self._trailing_gemm() and self.bias.numel() == self._N:
            # statistics, folding and the moving-average update in three launches (the folding algebra and its
            # gradient would otherwise be some forty elementwise launches on [N] vectors)
            mean, meansq, chained = self._batch_moments(inputs, raw=True, quant=quant, chain=True)
            if chained is not None:
                inputs = chained
            fold = (self._kernel.reshape(self._K, self._N), self.bias.reshape(-1), self.bn_gamma.reshape(-1) if self.scale else None,
                    mean, meansq, True, epsilon(), self.moving_mean.view(-1), self.moving_variance.view(-1), self.momentum)
            fk, fb = (_eligible(self.kq, self._kernel), _eligible(self.bq, self.bias)) if training is True else (None, None)
            if fk is not None and fb is not None:
                # folding and both quantizers in one launch each way
                qkernel, qbias = ops.bn_fold_quant(*fold, *((f._k.view(-1), f._i.view(-1), f._third().view(-1), f._mode(True)) for f in (fk, fb)))
                qkernel, qbias = qkernel.view(self._kernel.shape), qbias.view(self.bias.shape)
                # their gradients are read by the folding's backward and by nothing else, and it sums pending slices first:
                # the contraction may leave its kernel / bias gradient as slices for that launch
                qkernel._hgq_single_use = qbias._hgq_single_use = True
            else:
                fused_kernel, fused_bias = ops.bn_fold(*fold)
                # kernel and bias quantizers in one launch each way (they are a few thousand elements together)
                qkernel, qbias = quantize_together([(self.kq, fused_kernel.view(self._kernel.shape)),
                                                    (self.bq, fused_bias.view(self.bias.shape))], training)
        else:
            if training and self.trainable:
                mean, var = self._batch_moments(inputs)
                with torch.no_grad():
                    self.moving_mean.copy_(self.moving_mean * self.momentum + mean * (1.0 - self.momentum))
                    self.moving_variance.copy_(self.moving_variance * self.momentum + var * (1.0 - self.momentum))
            else:
                var, mean = self.moving_variance, self.moving_mean
            qkernel, qbias = self.get_fused_qkernel_and_qbias(training, mean, var)
        # an input quantized above is contracted as it is; otherwise the contraction quantizes it while staging
        # (and leaves the abs-max slices for the integer-bit update, as QEinsumDense does)
        enable_iq, self._enable_iq = self._enable_iq, quant is not None
        try:
            if then is not None:  # the mean over the middle axis that follows, taken with the contraction where the kernels cover it
                return self._finish_then(*self._contract(inputs, qkernel, qbias, training, mean_rows=inputs.shape[1]), then)
            y, act_done = self._contract(inputs, qkernel, qbias, training)
        finally:
            self._enable_iq = enable_iq
        if self.activation is not None and not act_done:
            y = self.activation(y)
        return y

    call._takes_then = True
