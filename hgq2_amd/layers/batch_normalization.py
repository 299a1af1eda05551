"""QBatchNormalization (reference src/hgq/layers/batch_normalization.py:10-206): batch normalisation as
a quantized per-channel affine map

    y = iq(x) * kq(scale) + bq(offset),   scale = gamma / sqrt(var + epsilon),   offset = beta - mean * scale

with the batch moments in training (moving averages updated in place) and the moving moments otherwise.
The layer's own ``epsilon`` is used (not the global one), and with ``center=False`` the reference puts 1 in
the place of ``bn_beta`` (:117-120, :145-148); both are kept.  EBOPs ``sum(bits_in * bits_scale) +
mean(bits_offset) * size``.  The moments over a trailing channel axis come from the one-pass column-moment
kernel (``hgq_col_moments_fwd / _bwd``); in a training step scale, offset, the moving-average updates and the two
quantizers are one launch each way (``_fold_in_one_launch``)."""

from __future__ import annotations

from math import prod

import torch

from .. import ops
from ..core import get_initializer
from ..quantizer import Quantizer, QuantizerConfig
from ..quantizer.prefetch import _eligible, quantize_together
from .core.base import QLayerBaseSingleInput, mean_bits


class QBatchNormalization(QLayerBaseSingleInput):
    def __init__(self, axis=-1, momentum=0.99, epsilon=1e-3, center=True, scale=True, beta_initializer='zeros',
                 gamma_initializer='ones', moving_mean_initializer='zeros', moving_variance_initializer='ones',
                 beta_regularizer=None, gamma_regularizer=None, beta_constraint=None, gamma_constraint=None, synchronized=False,
                 kq_conf: None | QuantizerConfig = None, iq_conf: None | QuantizerConfig = None,
                 bq_conf: None | QuantizerConfig = None, **kwargs):
        super().__init__(iq_conf=iq_conf, **kwargs)
        self.axis, self.momentum, self.epsilon = int(axis), float(momentum), float(epsilon)
        self.center, self.scale, self.synchronized = bool(center), bool(scale), synchronized
        self.beta_initializer, self.gamma_initializer = get_initializer(beta_initializer), get_initializer(gamma_initializer)
        self.moving_mean_initializer = get_initializer(moving_mean_initializer)
        self.moving_variance_initializer = get_initializer(moving_variance_initializer)
        self.beta_regularizer, self.gamma_regularizer = beta_regularizer, gamma_regularizer
        self.beta_constraint, self.gamma_constraint = beta_constraint, gamma_constraint
        self._kq = Quantizer(kq_conf or QuantizerConfig('default', 'weight'), name=f'{self.name}_kq')
        self._bq = Quantizer(bq_conf or QuantizerConfig('default', 'bias'), name=f'{self.name}_bq')
        self.bn_gamma = self.bn_beta = None

    @property
    def kq(self):
        return self._kq

    @property
    def bq(self):
        return self._bq

    def build(self, input_shape):
        super().build(input_shape)
        input_shape = tuple(input_shape)
        if self.axis < 0:
            self.axis += len(input_shape)
        channels = (int(input_shape[self.axis]),)
        if self.scale:
            self.bn_gamma = self.add_weight(shape=channels, name='bn_gamma', initializer=self.gamma_initializer,
                                            regularizer=self.gamma_regularizer, constraint=self.gamma_constraint)
        if self.center:
            self.bn_beta = self.add_weight(shape=channels, name='bn_beta', initializer=self.beta_initializer,
                                           regularizer=self.beta_regularizer, constraint=self.beta_constraint)
        self.moving_mean = self.add_weight(shape=channels, name='moving_mean', initializer=self.moving_mean_initializer, trainable=False)
        self.moving_variance = self.add_weight(shape=channels, name='moving_variance', initializer=self.moving_variance_initializer,
                                               trainable=False)
        for q in (self._bq, self._kq):
            q._build_device = self._build_device
            q.build(channels)
            q.built = True
        self._reduction_axes = tuple(a for a in range(len(input_shape)) if a != self.axis)
        shape = [1] * len(input_shape)
        shape[self.axis] = channels[0]
        self._shape = tuple(shape)

    def _moments(self, x):
        """Mean and biased variance ``mean(x**2) - mean(x)**2`` over all axes but the channel axis."""
        if x.is_cuda and self.axis == x.dim() - 1 and x.dtype == torch.float32 and x.numel() > 0:
            mean, meansq = ops.col_moments(x.reshape(-1, x.shape[-1]).contiguous())  # one pass over x
        else:
            mean = torch.mean(x, dim=self._reduction_axes)
            meansq = torch.mean(torch.square(x), dim=self._reduction_axes)
        return mean, meansq - torch.square(mean)

    def _scale_offset(self, mean, variance):
        bn_gamma = self.bn_gamma if self.scale else 1
        bn_beta = self.bn_beta if self.center else 1
        scale = bn_gamma / torch.sqrt(variance + self.epsilon)
        return scale, bn_beta - mean * scale

    @property
    def qscaler_and_qoffset(self):
        scale, offset = self._scale_offset(self.moving_mean, self.moving_variance)
        return self.kq(scale, training=False), self.bq(offset, training=False)

    def call(self, inputs, training=None, mask=None):
        if mask is not None:
            raise NotImplementedError('QBatchNormalization: masked moments are not supported')
        if self.enable_iq:
            inputs = self.iq(inputs, training=training)
        fused = self._fold_in_one_launch(inputs) if training is True else None
        if fused is not None:
            qscale, qoffset = fused
            return ops.affine_rows(inputs, qscale.reshape(self._shape), qoffset.reshape(self._shape))
        if training:
            mean, variance = self._moments(inputs)
            with torch.no_grad():
                self.moving_mean.copy_(self.moving_mean * self.momentum + mean * (1.0 - self.momentum))
                self.moving_variance.copy_(self.moving_variance * self.momentum + variance * (1.0 - self.momentum))
        else:
            mean, variance = self.moving_mean, self.moving_variance
        scale, offset = self._scale_offset(mean, variance)
        qscale, qoffset = quantize_together([(self.kq, scale.contiguous()), (self.bq, offset.contiguous())], training)
        qscale, qoffset = qscale.reshape(self._shape), qoffset.reshape(self._shape)
        return ops.affine_rows(inputs, qscale, qoffset)

    def _fold_in_one_launch(self, x):
        """``(kq(scale), bq(offset))`` of a training step from the batch moments in ONE launch each way - scale, offset,
        the moving-average updates and both quantizers (``hgq_bn_fold_quant_fwd / _bwd`` on a kernel of ones: a folded
        kernel ``1 * scale`` and a folded bias ``beta - mean * scale`` are exactly this layer's two operands) - instead
        of some twenty launches on [channels] vectors; ``None`` where the kernels do not apply."""
        if not (x.is_cuda and x.dtype == torch.float32 and self.axis == x.dim() - 1 and x.numel() > 0):
            return None
        fk, fb = _eligible(self.kq, self.moving_mean), _eligible(self.bq, self.moving_mean)
        if fk is None or fb is None:
            return None
        C = x.shape[-1]
        ones = self.__dict__.get('_ones')
        if ones is None or ones.device != x.device or ones.numel() != C:
            ones = torch.ones(1, C, dtype=torch.float32, device=x.device)
            object.__setattr__(self, '_ones', ones)
        mean, meansq = ops.col_moments(x.reshape(-1, C).contiguous())  # one pass over x
        beta = self.bn_beta if self.center else ones.view(-1)  # (the reference puts 1 in the place of a missing beta)
        qs, qo = ops.bn_fold_quant(ones, beta, self.bn_gamma if self.scale else None, mean, meansq, True, self.epsilon,
                                   self.moving_mean, self.moving_variance, self.momentum,
                                   *((f._k.view(-1), f._i.view(-1), f._third().view(-1), f._mode(True)) for f in (fk, fb)))
        return qs.view(-1), qo

    def _compute_ebops(self, shape):
        bw_inp = self.iq.bits_(shape)
        bw_ker = self.kq.bits_(self.moving_mean.shape).reshape(self._shape)
        bw_bias = self.bq.bits_(self.moving_mean.shape).reshape(self._shape)
        return torch.sum(bw_inp * bw_ker) + mean_bits(bw_bias) * float(prod(shape))

    def compute_output_shape(self, input_shape):
        return input_shape

    def get_config(self):
        config = super().get_config()
        config.update(axis=self.axis, momentum=self.momentum, epsilon=self.epsilon, center=self.center, scale=self.scale,
                      kq_conf=self.kq.config, bq_conf=self.bq.config)
        return config
