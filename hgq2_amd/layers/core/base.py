"""Base classes of the quantized layers.

Follows reference src/hgq/layers/core/base.py: the ``call`` wrapper that computes EBOPs, adds
``ebops * beta`` to the loss and applies the output quantizer (``QLayerMeta.__call__``, :57-116),
``QLayerBase`` (:119-243), ``QLayerBaseSingleInput`` (:246-272), ``MultipleQuantizers`` (:275-301),
``QLayerBaseMultiInputs`` (:304-352).
"""

from __future__ import annotations

from collections.abc import Iterable, Sequence

import torch
from torch import nn

from ...config.layer import global_config
from ...core import Constant, Initializer, Layer
from ...quantizer import Quantizer, QuantizerConfig


def scale_ebops(ebops: torch.Tensor, parallelization_factor, n_parallel) -> torch.Tensor:
    """``ebops * parallelization_factor / n_parallel`` as the reference evaluates it (src/hgq/layers/core/dense.py:80,
    pooling.py:30): a product, then a correctly rounded fp32 division.  On the GPU torch divides by a Python number with a
    reciprocal multiply, which can land one ulp low - and the uint32 cast of the estimate one count low - so the divisor
    goes in as a tensor."""
    ebops = ebops * float(parallelization_factor)
    if float(n_parallel) == 1.0:
        return ebops
    return ebops / torch.full((), float(n_parallel), dtype=ebops.dtype, device=ebops.device)


def mean_bits(bits: torch.Tensor) -> torch.Tensor:
    """``mean(bits)`` as a sum and one correctly rounded division (the library's GPU mean multiplies by a rounded 1 / n)."""
    return torch.sum(bits) / torch.full((), float(bits.numel()), dtype=bits.dtype, device=bits.device)


class QLayerBase(Layer):
    """Handles the input / output quantizers, the ``beta`` and ``ebops`` variables and the
    EBOPs loss term.  Subclasses implement ``call`` and ``_compute_ebops(*input_shapes)``."""

    __output_quantizer_handled__ = False

    def __init__(self, enable_ebops=None, beta0=None, enable_oq=None, enable_iq=None, oq_conf=None,
                 ebops_factor: float = 1.0, **kwargs):
        super().__init__(**kwargs)
        # arguments left at None take the scope's defaults (config.layer.global_config)
        def scoped(value, key):
            return global_config[key] if value is None else value

        start = scoped(beta0, 'beta0')
        self._beta0 = start if isinstance(start, Initializer) else Constant(float(start))
        self._enable_iq, self._enable_oq = scoped(enable_iq, 'enable_iq'), scoped(enable_oq, 'enable_oq')
        # the resource estimate needs the input bit-widths: without an input quantizer it is off unless asked for
        self._enable_ebops = (global_config['enable_ebops'] and self._enable_iq) if enable_ebops is None else enable_ebops
        self.ebops_factor = ebops_factor
        self._beta = self._ebops = None
        if self._enable_oq:
            self._oq = Quantizer(oq_conf if oq_conf else QuantizerConfig('default', 'datalane'), name=f'{self.name}_oq')

    @property
    def enable_iq(self):
        return self._enable_iq

    @property
    def enable_oq(self):
        return self._enable_oq

    @property
    def oq(self):
        if not self.enable_oq:
            raise AttributeError(f'{self.name} was built without an output quantizer (enable_oq=False)')
        return self._oq

    @property
    def beta(self):
        if self._beta is None:
            return torch.zeros(())
        return self._beta

    @property
    def ebops(self):
        if self._ebops is None:
            return torch.zeros((), dtype=torch.int64)
        return self._ebops

    @property
    def enable_ebops(self):
        return self._enable_ebops

    def build(self, input_shape=None):
        if self.enable_ebops and self._beta is None:
            self._beta = self.add_weight(name='beta', shape=(), initializer=self._beta0, trainable=False)
            self._ebops = self.add_weight(name='ebops', shape=(), initializer=Constant(0.0), trainable=False, dtype='uint32')
        self.built = True
        if not self.enable_oq or self.oq.built:
            return
        self.try_build_output_quantizer(input_shape)

    def try_build_output_quantizer(self, input_shape=None):
        try:
            output_shape = self.compute_output_shape(input_shape)
        except Exception:
            return
        self.oq._build_device = self._build_device
        self.oq.build(tuple(output_shape))
        self.oq.built = True

    def _ebops_loss_term(self, *shapes):
        """``ebops = _compute_ebops(...) * ebops_factor; _ebops.assign(cast(ebops, uint32))``; returns
        the loss term ``ebops * beta`` (reference :101-104).  Layers with a fused kernel override this."""
        ebops = self._compute_ebops(*shapes)
        if ebops.is_cuda and ebops.dtype == torch.float32 and ebops.numel() == 1 and self._beta.dtype == torch.float32:
            from ... import ops

            return ops.ebops_finish(ebops, self.ebops_factor, self._beta, self._ebops)  # one launch instead of five
        ebops = ebops * self.ebops_factor
        with torch.no_grad():
            self._ebops.view(torch.int32).copy_(ebops.detach().to(torch.int64).to(torch.int32))
        return ebops * self._beta

    def _wrapped_call(self, *args, training=None, **kwargs):
        self._oq_applied_in_call = False  # a `call` that ran the output quantizer in a fused kernel sets this
        r = self.call(*args, training=training, **kwargs)
        if (training or training == 'tracing') and self.enable_ebops:
            tensors = args[0] if isinstance(args[0], (tuple, list)) else [a for a in args if isinstance(a, torch.Tensor)]
            shapes = [(1,) + tuple(t.shape[1:]) for t in tensors]
            self.add_loss(self._ebops_loss_term(*shapes))
        self._finish_call()
        if not self.enable_oq or self.__output_quantizer_handled__ or self._oq_applied_in_call:
            return r
        if isinstance(r, (tuple, list)):
            raise AssertionError(f'{type(self).__name__} {self.name!r} returned {len(r)} outputs: a layer with several outputs '
                                 'applies its output quantizers itself (__output_quantizer_handled__)')
        return self.oq(r, training=training)

    def _finish_call(self):
        """Hook: state updates a layer deferred so they could be fused with the EBOPs kernel."""

    def get_config(self):
        return {
            'name': self.name,
            'enable_ebops': self.enable_ebops,
            'ebops_factor': self.ebops_factor,
            'beta0': self._beta0,
            'enable_oq': self.enable_oq,
            'enable_iq': self.enable_iq,
            'oq_conf': self.oq.config if self.enable_oq else None,
        }

    def _compute_ebops(self, *args, **kwargs):
        raise NotImplementedError(f'{type(self).__name__} does not define its EBOPs estimate')


class QLayerBaseSingleInput(QLayerBase):
    def __init__(self, iq_conf: QuantizerConfig | None = None, **kwargs):
        super().__init__(**kwargs)
        if self._enable_iq:
            self._iq = Quantizer(iq_conf if iq_conf else QuantizerConfig('default', 'datalane'), name=f'{self.name}_iq')

    @property
    def iq(self):
        if not self.enable_iq:
            raise AttributeError(f'{self.name} was built without an input quantizer (enable_iq=False)')
        return self._iq

    def build(self, input_shape=None):
        super().build(input_shape)
        if self.enable_iq and not self._iq.built:
            self.iq._build_device = self._build_device
            self.iq.build(tuple(input_shape))
            self.iq.built = True

    def get_config(self):
        config = super().get_config()
        config['iq_conf'] = self.iq.config if self.enable_iq else None
        return config


class MultipleQuantizers(Layer):
    """One quantizer per input of a layer that takes several; behaves as the sequence of them."""

    def __init__(self, configs: Sequence[QuantizerConfig], **kwargs):
        super().__init__(**kwargs)
        self.quantizers = nn.ModuleList([Quantizer(c) for c in configs])

    def call(self, x, training=None):
        if len(x) != len(self.quantizers):
            raise AssertionError(f'{self.name}: {len(self.quantizers)} quantizers for {len(x)} inputs')
        return tuple(q(t, training=training) for q, t in zip(self.quantizers, x))

    def build(self, shapes):
        for shape, q in zip(shapes, self.quantizers):
            q._build_device = self._build_device
            q.build(tuple(shape))
            q.built = True
        self.built = True

    def __len__(self):
        return len(self.quantizers)

    def __bool__(self):
        return len(self) != 0

    def __iter__(self):
        return iter(self.quantizers)

    def __getitem__(self, index):
        return self.quantizers[index]


class QLayerBaseMultiInputs(QLayerBase):
    def __init__(self, iq_confs=None, **kwargs):
        super().__init__(**kwargs)
        if self.enable_iq:
            self._iq_confs = iq_confs if iq_confs is not None else QuantizerConfig('default', 'datalane')

    @property
    def iq(self):
        if not self.enable_iq:
            raise AttributeError(f'{self.name} was built without input quantizers (enable_iq=False)')
        if not self.built:
            raise AttributeError(f'{self.name}: the input quantizers exist once the layer is built (one per input)')
        return self._iq

    @property
    def iq_confs(self):
        assert self.enable_iq, f'{self.name} has no input quantizers, hence no iq_confs'
        return self._iq_confs

    def build(self, input_shape=None):
        super().build(input_shape)
        if not self.enable_iq:
            return
        for shape in input_shape:
            assert isinstance(shape, Iterable), f'{self.name}: input_shape must list one shape per input, found {shape!r}'
        if isinstance(self._iq_confs, QuantizerConfig):  # one configuration for every input
            self._iq_confs = [self._iq_confs for _ in input_shape]
        assert len(self._iq_confs) == len(input_shape), f'{self.name}: {len(self._iq_confs)} iq_confs for {len(input_shape)} inputs'
        self._iq = MultipleQuantizers(self._iq_confs)
        self._iq._build_device = self._build_device
        self._iq.build(input_shape)
