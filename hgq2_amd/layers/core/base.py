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
        beta0 = beta0 if beta0 is not None else global_config['beta0']
        beta0 = Constant(float(beta0)) if not isinstance(beta0, Initializer) else beta0
        self._enable_iq = enable_iq if enable_iq is not None else global_config['enable_iq']
        self._enable_oq = enable_oq if enable_oq is not None else global_config['enable_oq']
        if enable_ebops is None:
            enable_ebops = global_config['enable_ebops'] and self.enable_iq
        self._enable_ebops = enable_ebops
        self._beta0 = beta0
        self.ebops_factor = ebops_factor
        self._beta = None
        self._ebops = None
        if self.enable_oq:
            oq_conf = oq_conf or QuantizerConfig('default', 'datalane')
            self._oq = Quantizer(oq_conf, name=f'{self.name}_oq')

    @property
    def enable_iq(self):
        return self._enable_iq

    @property
    def enable_oq(self):
        return self._enable_oq

    @property
    def oq(self):
        if not self.enable_oq:
            raise AttributeError(f'oq has been disabled for {self.name}.')
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
        assert not isinstance(r, (tuple, list)), (
            f'Layer {self.name}({type(self)}) returns multiple outputs, which must be handled in subclasses.'
        )
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
        raise NotImplementedError('This method is abstract and should be implemented in subclasses.')


class QLayerBaseSingleInput(QLayerBase):
    def __init__(self, iq_conf: QuantizerConfig | None = None, **kwargs):
        super().__init__(**kwargs)
        if self.enable_iq:
            iq_conf = iq_conf or QuantizerConfig('default', 'datalane')
            self._iq = Quantizer(iq_conf, name=f'{self.name}_iq')

    @property
    def iq(self):
        if not self.enable_iq:
            raise AttributeError(f'iq has been disabled for {self.name}.')
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
    def __init__(self, configs: Sequence[QuantizerConfig], **kwargs):
        super().__init__(**kwargs)
        self.quantizers = nn.ModuleList(Quantizer(config) for config in configs)

    def call(self, x, training=None):
        assert len(self) == len(x), f'{self.name} ({self.__class__.__name__}) expects {len(self)} inputs, got {len(x)}.'
        return tuple(f(x_, training=training) for f, x_ in zip(self.quantizers, x))

    def build(self, shapes):
        for q, shape in zip(self.quantizers, shapes):
            q._build_device = self._build_device
            q.build(tuple(shape))
            q.built = True
        self.built = True

    def __bool__(self):
        return len(self.quantizers) > 0

    def __len__(self):
        return len(self.quantizers)

    def __getitem__(self, item):
        return self.quantizers[item]

    def __iter__(self):
        return iter(self.quantizers)


class QLayerBaseMultiInputs(QLayerBase):
    def __init__(self, iq_confs=None, **kwargs):
        super().__init__(**kwargs)
        if self.enable_iq:
            self._iq_confs = iq_confs if iq_confs is not None else QuantizerConfig('default', 'datalane')

    @property
    def iq(self):
        if not self.enable_iq:
            raise AttributeError(f'iq has been disabled for {self.name}.')
        if not self.built:
            raise AttributeError(f'iqs is not available before build for {self.name}.')
        return self._iq

    @property
    def iq_confs(self):
        assert self.enable_iq, f'iq_confs has been disabled for {self.name}.'
        return self._iq_confs

    def build(self, input_shape=None):
        super().build(input_shape)
        if not self.enable_iq:
            return
        n_input = len(input_shape)
        for s in input_shape:
            assert isinstance(s, Iterable), f'each element of input_shape must be iterable, got {s}'
        if isinstance(self.iq_confs, QuantizerConfig):
            self._iq_confs = [self.iq_confs] * n_input
        assert len(self.iq_confs) == n_input, (
            f'number of iq_confs must match number of inputs, got {len(self._iq_confs)} != {n_input}'
        )
        self._iq = MultipleQuantizers(self._iq_confs)
        self._iq._build_device = self._build_device
        self._iq.build(input_shape)
