"""QSoftmax (reference src/hgq/layers/softmax.py:13-217): the bit-accurate, table-driven softmax

    d = max(x) - x;  e = oq_exp(exp(-iq_exp(d) * input_scaler));  s = sum(e);
    r = oq_inv(1 / (iq_inv(s) + epsilon));  y = oq(e * r)

whose exp and 1/x stages are functions of a few-bit argument (lookup tables in hardware).
"""

from __future__ import annotations

from collections.abc import Sequence
from math import prod

import torch

from .. import _lib, ops
from ..config.layer import global_config
from ..core import epsilon
from ..quantizer import QuantizerConfig
from ..quantizer.internal import FixedPointQuantizerKBI, FixedPointQuantizerKIF
from ..quantizer.internal.base import bw_layout
from .activation import QUnaryFunctionLUT
from .core.base import QLayerBaseSingleInput


FUSED = True  # module switch: False forces the per-stage path (used to cross-check the one-pass kernels)


class QSoftmax(QLayerBaseSingleInput):
    def __init__(self, axis: int | Sequence[int] | None = None, iq_conf: None | QuantizerConfig = None, stable=True,
                 enable_iq: None | bool = False, exp_iq_conf: None | QuantizerConfig = None,
                 exp_oq_conf: None | QuantizerConfig = None, inv_iq_conf: None | QuantizerConfig = None,
                 inv_oq_conf: None | QuantizerConfig = None, allow_heterogeneous_table: bool = False,
                 input_scaler: float = 1.0, parallelization_factor: int = -1, enable_ebops: None | bool = None, **kwargs):
        axes = kwargs.pop('axes', None)
        assert axis is None or axes is None, 'Use only one of `axis` or `axes`.'
        self.axes = axes or (tuple(axis) if isinstance(axis, Sequence) else (axis,) if axis is not None else (-1,))
        if enable_ebops is None:
            enable_ebops = global_config['enable_ebops']
        super().__init__(iq_conf=iq_conf, enable_iq=enable_iq, enable_ebops=enable_ebops, **kwargs)
        self.stable = stable
        self.parallelization_factor = parallelization_factor
        self._allow_heterogeneous_table = allow_heterogeneous_table
        self.input_scaler = input_scaler

        def _inv(x):
            return 1.0 / (x + epsilon())

        def _exp(x):
            if self.stable:
                return torch.exp(-x * self.input_scaler)
            return torch.exp(x * self.input_scaler)

        inv_iq_conf = inv_iq_conf or QuantizerConfig('default', 'datalane')
        exp_iq_conf = exp_iq_conf or QuantizerConfig('default', 'datalane')
        exp_oq_conf = exp_oq_conf or QuantizerConfig('default', 'table')
        inv_oq_conf = inv_oq_conf or QuantizerConfig('default', 'table')
        if not self._allow_heterogeneous_table:
            for conf in (inv_iq_conf, exp_iq_conf):
                conf.config['heterogeneous_axis'] = ()
                conf.config['homogeneous_axis'] = None
        for conf in (inv_oq_conf, exp_oq_conf):
            if 'k0' in conf.config:
                conf.config['k0'] = 0
            conf.config['overflow_mode'] = 'SAT'
            conf.config['round_mode'] = 'RND_CONV'

        self.inv_table = QUnaryFunctionLUT(
            _inv, inv_iq_conf, inv_oq_conf, enable_iq=True, enable_oq=True,
            allow_heterogeneous_table=allow_heterogeneous_table, name=f'{self.name}_inv_table',
            enable_ebops=self.enable_ebops, beta0=self._beta0.clone())
        self.exp_table = QUnaryFunctionLUT(
            _exp, exp_iq_conf, exp_oq_conf, enable_iq=self.stable, enable_oq=True,
            allow_heterogeneous_table=allow_heterogeneous_table, allow_heterogeneous_input=True,
            name=f'{self.name}_exp_table', enable_ebops=self.enable_ebops and stable, beta0=self._beta0.clone())
        self.supports_masking = True

    def get_config(self):
        config = super().get_config()
        config.update({'axes': tuple(self.axes), 'stable': self.stable, 'exp_oq_conf': self.exp_table.oq.config,
                       'exp_iq_conf': self.exp_table.iq.config if self.stable else None,
                       'inv_oq_conf': self.inv_table.oq.config, 'inv_iq_conf': self.inv_table.iq.config,
                       'allow_heterogeneous_table': self._allow_heterogeneous_table, 'input_scaler': self.input_scaler,
                       'parallelization_factor': self.parallelization_factor})
        return config

    def build(self, input_shape):
        self.exp_table._build_device = self._build_device
        self.exp_table.build(tuple(input_shape))
        self.exp_table.built = True
        self.axes = tuple(sorted(i if i >= 0 else i + len(input_shape) for i in self.axes))
        inv_shape = list(input_shape)
        for i in self.axes:
            inv_shape[i] = 1
        self.inv_table._build_device = self._build_device
        self.inv_table.build(tuple(inv_shape))
        self.inv_table.built = True
        super().build(input_shape)

    # ---- fused kernel path
    @staticmethod
    def _fusable_quantizer(q, training, shared: bool):
        """``(k, i, fb, mode, track)`` if the kernel can run this quantizer in place, else ``None``."""
        if q is None or not q.plain:
            return None
        inner = q.quantizer
        if not isinstance(inner, (FixedPointQuantizerKIF, FixedPointQuantizerKBI)) or not inner.built:
            return None
        if shared and inner._i.numel() != 1:
            return None
        if inner.stochastic and training is True:
            return None  # stochastic rounding draws in its own kernel
        track = False
        if inner.overflow_mode == 'WRAP' and inner.trainable:
            if training == 'tracing' or (training and not isinstance(inner, FixedPointQuantizerKIF)):
                return None  # calibration and the KBI tracking rule keep their own call sequence
            track = training is True
        return inner._k.view(-1), inner._i.view(-1), inner._third().view(-1), inner._mode(training is True), track

    def _fused_plan(self, x, training, mask):
        """Descriptors for ``ops.qsoftmax`` when this call maps onto the one-pass kernel, else ``None``."""
        if not (FUSED and self.stable and mask is None and x.is_cuda and x.dtype == torch.float32 and x.dim() >= 2):
            return None
        if self.axes != (x.dim() - 1,) or not 1 <= x.shape[-1] <= 256 or x.numel() == 0:
            return None
        if training not in (True, False, None):
            return None
        e, v = self.exp_table, self.inv_table
        if not (e.enable_iq and e.enable_oq and v.enable_iq and v.enable_oq):
            return None
        qs = [self._fusable_quantizer(q, training, True) for q in (e.iq, e.oq, v.iq, v.oq)]
        if any(q is None for q in qs):
            return None
        if self.enable_oq:
            if not self.oq.built:
                return None
            qo = self._fusable_quantizer(self.oq, training, False)
            layout = bw_layout(self.oq.quantizer._i.shape, x.shape)
            if qo is None or layout is None or layout[1] != 1 or layout[0] % x.shape[-1] != 0:
                return None
            qs.append(qo)
        else:
            qs.append(None)
        L = x.shape[-1]
        bw_rows = qs[4][1].numel() // L if qs[4] is not None else 1
        if _lib.load().hgq_qsoftmax_bwd_workspace(x.numel() // L, L, bw_rows, int(qs[4] is not None)) < 0:
            return None  # a row layout outside the kernel family
        return qs

    def _call_fused(self, x, training, qs, attention=None, attention_mask=None):
        e, v = self.exp_table, self.inv_table
        owners = (e.iq, e.oq, v.iq, v.oq, self.oq if self.enable_oq else None)
        track_mask = sum(bit for bit, q in zip((1, 0, 2, 0, 4), qs) if q is not None and q[4])
        descs = [None if q is None else q[:4] for q in qs]
        if attention is not None:  # scores and probabilities stay inside the kernel; y is the combined output
            mask, causal = attention_mask if attention_mask is not None else (None, False)  # masks are applied inside the kernel
            y, a1, a3, ao = ops.qattention(*attention, descs, self.input_scaler, epsilon(), track_mask, mask=mask, causal=causal)
        else:
            y, a1, a3, ao = ops.qsoftmax(x, descs, self.input_scaler, epsilon(), track_mask)
        for amax, n in ((a1, 0), (a3, 2), (ao, 4)):
            if amax.numel():
                owners[n].quantizer._track(amax, True)
        # what the two table layers' own call wrappers do after their call (EBOPs term, uint32 variable)
        accum_shape = tuple(x.shape[:-1]) + (1,)
        for table, shape in ((e, tuple(x.shape)), (v, accum_shape)):
            table._losses = []
            if training and table.enable_ebops:
                table.add_loss(table._ebops_loss_term((1,) + shape[1:]))
        return y

    def attention_plan(self, query, key, value, training):
        """Whether ``self(stand_in, attention=(query, key, value))`` can run scores, softmax and combine as one kernel;
        returns the shape-only stand-in for the scores, or ``None``."""
        if self.enable_iq or not query.is_cuda or query.dim() != 4:
            return None
        B, T, N, _ = query.shape
        stand_in = query.new_empty(()).expand(B, N, T, key.shape[1])
        qs = self._fused_plan(stand_in, training, None)
        if qs is None:
            return None
        entries = qs[4][1].numel() if qs[4] is not None else 0
        inner = self.oq.quantizer if qs[4] is not None else None
        saturates = inner is not None and (inner.overflow_mode != 'WRAP' or isinstance(inner, FixedPointQuantizerKBI))
        return stand_in if ops.qattention_supported(query, key, value, entries, saturates) else None

    def call(self, inputs, training=None, mask=None, attention=None, attention_mask=None):
        if attention is not None:  # `inputs` carries the shape of the scores only (see attention_plan)
            self._oq_applied_in_call = self.enable_oq
            return self._call_fused(inputs, training, self._fused_plan(inputs, training, None), attention, attention_mask)
        if self.enable_iq:
            inputs = self.iq(inputs, training=training)
        qs = self._fused_plan(inputs, training, mask)
        if qs is not None:
            self._oq_applied_in_call = self.enable_oq  # the kernel runs the output quantizer itself
            return self._call_fused(inputs, training, qs)
        if self.stable:
            if mask is not None:
                mask = mask.to(inputs.dtype)
                inputs = mask * inputs - (1 - mask) * 1e9
            inputs = torch.amax(inputs, dim=self.axes, keepdim=True) - inputs
        exp_inp = self.exp_table(inputs, training=training)
        if mask is not None:
            exp_inp = mask.to(inputs.dtype) * exp_inp
        sums = torch.sum(exp_inp, dim=self.axes, keepdim=True)
        divisor = self.inv_table(sums, training=training)
        return exp_inp * divisor

    def _ebops_loss_term(self, shape):
        # the stable form over the last axis: one launch for value, uint32 variable, loss term and gradients
        shape = tuple(shape)
        if self.stable and self.axes == (len(shape) - 1,) and self._beta is not None and self._beta.is_cuda:
            rows, L = prod(shape[:-1]), shape[-1]
            sub = self.iq if self.enable_iq else self.exp_table.iq
            operands = [sub.bits_operand(shape), self.exp_table.oq.bits_operand(shape),
                        self.inv_table.oq.bits_operand(shape[:-1] + (1,))]
            if all(op is not None for op in operands) and 0 < rows <= 2048 and rows * L < 2**31 and sum(op[3] for op in operands) <= 30720:
                n_instance = self.parallelization_factor if self.parallelization_factor > 0 else rows
                return ops.bits_ebops('softmax', operands, (rows, L, n_instance / rows, float(self.ebops_factor)), self._beta,
                                      self._ebops)
        return super()._ebops_loss_term(shape)

    def _compute_ebops(self, shape):
        accum_shape = tuple(1 if i in self.axes else s for i, s in enumerate(shape))
        max_instance = prod(accum_shape)
        n_instance = self.parallelization_factor if self.parallelization_factor > 0 else max_instance
        factor = n_instance / max_instance
        inp_bits = self.iq.bits_(shape) if self.enable_iq else 0
        exp_bits = self.exp_table.oq.bits_(shape)
        inv_bits = self.inv_table.oq.bits_(accum_shape)
        if self.stable:
            substract_ebops = torch.sum(inp_bits) if self.enable_iq else torch.sum(self.exp_table.iq.bits_(shape))
        else:
            substract_ebops = 0
        accum_ebops = torch.sum(exp_bits) - torch.sum(torch.amin(exp_bits, dim=self.axes))
        mult_ebops = torch.sum(exp_bits * inv_bits)
        ebops = substract_ebops + accum_ebops + mult_ebops
        if not self.stable:
            ebops = ebops + torch.sum((2.0**inp_bits) * exp_bits) * 1e-4
        return ebops * factor

    def compute_output_shape(self, input_shape):
        return input_shape

    @property
    def ebops(self):
        total = int(self._ebops.cpu().view(torch.int32)) if self._ebops is not None else 0
        for t in (self.exp_table, self.inv_table):
            if t._ebops is not None:
                total += int(t._ebops.cpu().view(torch.int32))
        return total
