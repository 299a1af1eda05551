"""Minimal layer runtime the API mirror sits on (Keras v3 is not required on the host).

It reproduces the few Keras behaviours the hot path relies on:

* lazy ``build(input_shape)`` on first call and ``add_weight(...)`` with per-variable
  ``constraint`` / ``regularizer`` / ``trainable``;
* the ``training`` flag is inherited by nested layer calls through a call context, so
  ``self.kq(self._kernel)`` inside a layer sees the outer call's flag;
* ``add_loss`` terms are collected per top-level call; variable regularizers are summed into
  the loss; constraints are applied after the optimizer update.
"""

from __future__ import annotations

import math
import threading
from typing import Any

import numpy as np
import torch
from torch import nn

_ctx = threading.local()

EPSILON = 1e-7  # keras.backend.epsilon() default


def epsilon() -> float:
    return EPSILON


def _training_ctx():
    return getattr(_ctx, 'training', None)


class TrainingFlagWrapper:
    """Falsy object that compares equal to a string; used for ``training='tracing'``
    (reference src/hgq/utils/minmax_trace.py:24-32)."""

    def __init__(self, value):
        self.value = value

    def __bool__(self):
        return self.value is True

    def __eq__(self, other):
        return self.value == other

    def __hash__(self):
        return hash(self.value)


# ------------------------------------------------------------------------------------------
# initializers
# ------------------------------------------------------------------------------------------
class Initializer:
    def __call__(self, shape, dtype, device, generator=None):
        raise NotImplementedError

    def clone(self):
        return self


class Constant(Initializer):
    def __init__(self, value=0.0):
        self.value = value

    def __call__(self, shape, dtype, device, generator=None):
        return torch.full(tuple(shape), self.value, dtype=torch.float32).to(dtype).to(device)

    def clone(self):
        return Constant(self.value)

    def get_config(self):
        return {'value': self.value}


class GlorotUniform(Initializer):
    def __init__(self, seed=None):
        self.seed = seed

    def get_config(self):
        return {'seed': self.seed}

    def __call__(self, shape, dtype, device, generator=None):
        shape = tuple(shape)
        if len(shape) < 1:
            fan_in = fan_out = 1
        elif len(shape) == 1:
            fan_in = fan_out = shape[0]
        elif len(shape) == 2:
            fan_in, fan_out = shape
        else:  # conv kernels: receptive field * channels
            rf = int(np.prod(shape[:-2]))
            fan_in, fan_out = shape[-2] * rf, shape[-1] * rf
        limit = math.sqrt(6.0 / (fan_in + fan_out))
        g = generator
        if self.seed is not None:
            g = torch.Generator().manual_seed(self.seed)
        return ((torch.rand(shape, generator=g) * 2 - 1) * limit).to(dtype).to(device)


_INITIALIZERS = {
    'zeros': lambda: Constant(0.0),
    'ones': lambda: Constant(1.0),
    'glorot_uniform': lambda: GlorotUniform(),
}


def get_initializer(spec) -> Initializer:
    if isinstance(spec, Initializer):
        return spec
    if isinstance(spec, (int, float, np.number)):
        return Constant(float(spec))
    if isinstance(spec, str) and spec in _INITIALIZERS:
        return _INITIALIZERS[spec]()
    raise ValueError(f'unknown initializer {spec!r}')


_DTYPES = {'float32': torch.float32, 'uint8': torch.uint8, 'uint32': torch.uint32, 'int32': torch.int32, None: torch.float32}

_default_device = None


def set_default_device(device):
    """Device on which layers create their variables when built without seeing a tensor."""
    global _default_device
    _default_device = torch.device(device) if device is not None else None


def default_device():
    if _default_device is not None:
        return _default_device
    return torch.device('cuda', torch.cuda.current_device()) if torch.cuda.is_available() else torch.device('cpu')


_name_counts: dict[str, int] = {}


def base_name(cls_name: str) -> str:
    """``QDense`` -> ``q_dense``: the stem of a layer's automatic name."""
    return ''.join('_' + c.lower() if c.isupper() and i else c.lower() for i, c in enumerate(cls_name))


def _auto_name(cls_name: str) -> str:
    base = base_name(cls_name)
    n = _name_counts.get(base, 0)
    _name_counts[base] = n + 1
    return base if n == 0 else f'{base}_{n}'


# Top-level training calls run all kernel / bias quantizers of the model in one launch first (quantizer/prefetch.py).
PREFETCH_WEIGHT_QUANTIZERS = True


# Walking a module tree costs the host tens of microseconds per layer; a training step needs the walk three times
# (clearing the loss lists, collecting the weight quantizers, collecting loss terms and regularised variables).  The
# results are cached per root and keyed on this counter, which every change of a tree bumps: a layer gaining a
# sub-module or a variable, or being built.
TREE_EPOCH = [0]


class TreeCache:
    __slots__ = ('key', 'layers', 'quantized', 'regularised')


def _structure_changed(*_):
    TREE_EPOCH[0] += 1


# any module or parameter registered anywhere (an `nn.ModuleList.append` inside a custom layer, `register_parameter`)
# ends the validity of the cached lists; what these hooks cannot see - a regularizer attached to an existing parameter
# after the first step - needs `invalidate_tree_caches()`
torch.nn.modules.module.register_module_module_registration_hook(_structure_changed)
torch.nn.modules.module.register_module_parameter_registration_hook(_structure_changed)


def invalidate_tree_caches():
    """Call after changing a model in a way no registration shows: attaching or removing ``regularizer`` / ``constraint``
    attributes of existing parameters."""
    TREE_EPOCH[0] += 1


def tree_cache(root) -> TreeCache:
    """Lists of a module tree that a training step needs: its layers, the layers that declare kernel / bias quantizers,
    the trainable variables with a regularizer."""
    key = (TREE_EPOCH[0], len(root._modules))
    c = root.__dict__.get('_hgq_tree_cache')
    if c is None or c.key != key:
        c = TreeCache()
        c.key = key
        mods = list(root.modules())
        c.layers = [m for m in mods if isinstance(m, Layer)]
        c.quantized = [m for m in mods if hasattr(m, '_weight_quantizer_inputs')]
        c.regularised = [p for p in root.parameters() if getattr(p, 'regularizer', None) is not None]
        object.__setattr__(root, '_hgq_tree_cache', c)
    return c


class Layer(nn.Module):
    """Keras-like layer on top of ``torch.nn.Module``."""

    def __setattr__(self, name, value):
        if isinstance(value, (nn.Module, torch.Tensor)) or name == 'built':
            if isinstance(value, (nn.Module, nn.Parameter)) or name == 'built':
                TREE_EPOCH[0] += 1
            super().__setattr__(name, value)
            return
        d = self.__dict__
        if name in d.get('_parameters', ()) or name in d.get('_buffers', ()) or name in d.get('_modules', ()):
            super().__setattr__(name, value)  # e.g. `self.bias = None` for a registered parameter
            return
        object.__setattr__(self, name, value)  # plain per-call state (flags, shapes, pending work): no registration logic

    def __init__(self, name: str | None = None, trainable: bool = True, dtype: Any = None, **kwargs):
        super().__init__()
        if kwargs:
            raise TypeError(f'unexpected keyword arguments {sorted(kwargs)} for {type(self).__name__}')
        self.name = name or _auto_name(type(self).__name__)
        self._layer_trainable = trainable
        self.built = False
        self._losses: list[torch.Tensor] = []
        self._build_device = None

    # ---- variables
    @property
    def trainable(self):
        return self._layer_trainable

    def add_weight(self, name, shape=(), initializer='zeros', trainable=True, dtype=None, constraint=None,
                   regularizer=None, **_unused):
        dt = _DTYPES[dtype] if not isinstance(dtype, torch.dtype) else dtype
        device = self._build_device or default_device()
        value = get_initializer(initializer)(shape, dt, device)
        attr = f'_var_{name}'
        if dt.is_floating_point:
            p = nn.Parameter(value, requires_grad=bool(trainable) and self._layer_trainable)
            p.constraint = constraint
            p.regularizer = regularizer
            p.var_name = name
            self.register_parameter(attr, p)
            TREE_EPOCH[0] += 1
            return p
        self.register_buffer(attr, value)
        return getattr(self, attr)

    # ---- losses
    def add_loss(self, value):
        self._losses.append(value)

    @property
    def losses(self):
        """``add_loss`` terms of the last call of this layer and its sub-layers, plus the
        regularization losses of all variables."""
        out = []
        for m in self.modules():
            if isinstance(m, Layer):
                out += m._losses
        for p in self.parameters():
            r = getattr(p, 'regularizer', None)
            if r is not None and p.requires_grad:
                out.append(r(p))
        return out

    def _clear_losses(self):
        for m in tree_cache(self).layers:
            m.__dict__['_losses'] = []

    def apply_constraints(self):
        """What a Keras optimizer does after each update."""
        with torch.no_grad():
            for p in self.parameters():
                c = getattr(p, 'constraint', None)
                if c is not None and p.requires_grad:
                    p.copy_(c(p))

    # ---- build / call
    def build(self, input_shape=None):
        self.built = True

    def compute_output_shape(self, input_shape):
        return input_shape

    def _maybe_build(self, args):
        if self.built:
            return
        first = args[0]
        if isinstance(first, (tuple, list)) and len(first) and isinstance(first[0], torch.Tensor):
            self._build_device = first[0].device
            self.build([tuple(t.shape) for t in first])
        elif isinstance(first, torch.Tensor):
            self._build_device = first.device
            self.build(tuple(first.shape))
        else:
            self.build(None)
        self.built = True

    def __call__(self, *args, training=None, **kwargs):
        outer = _training_ctx()
        if training is None:
            training = outer if outer is not None else False
        top = getattr(_ctx, 'depth', 0) == 0
        if top:
            self._clear_losses()
            if training is True and self.built and PREFETCH_WEIGHT_QUANTIZERS:
                from .quantizer.prefetch import prefetch_weight_quantizers

                prefetch_weight_quantizers(self)
        else:
            self._losses = []
        _ctx.training = training
        _ctx.depth = getattr(_ctx, 'depth', 0) + 1
        if top:
            from . import ops

            ops.begin_deferred()  # single-workgroup launches that nothing in the forward waits for go out together at the end
            ops.advance_seed_generators()  # draw counters of stochastic rounding: the previous step's draws are behind them now
        ok = False
        try:
            if top and args and isinstance(args[0], torch.Tensor):
                self._last_input_shape = (None,) + tuple(args[0].shape[1:])
            self._maybe_build(args)
            out = self._wrapped_call(*args, training=training, **kwargs)
            ok = True
            return out
        finally:
            _ctx.depth -= 1
            _ctx.training = outer
            if top:
                ops.end_deferred(discard=not ok)

    def _wrapped_call(self, *args, training=None, **kwargs):
        return self.call(*args, training=training, **kwargs)

    def call(self, *args, **kwargs):
        raise NotImplementedError

    def forward(self, *args, **kwargs):  # nn.Module API
        return self(*args, **kwargs)

    def get_config(self):
        return {'name': self.name}

    @classmethod
    def from_config(cls, config):
        return cls(**config)

    def extra_repr(self):
        return f'name={self.name}'


class Sequential(Layer):
    def __init__(self, layers=(), **kwargs):
        super().__init__(**kwargs)
        self.layers = nn.ModuleList(list(layers))

    def add(self, layer):
        self.layers.append(layer)
        TREE_EPOCH[0] += 1

    def get_config(self):
        return {'name': self.name, 'layers': list(self.layers)}

    def build(self, input_shape=None):
        self.built = True

    def call(self, x, training=None):
        layers, k = list(self.layers), 0
        while k < len(layers):
            layer = layers[k]
            nxt = layers[k + 1] if k + 1 < len(layers) else None
            absorbs = getattr(layer, 'absorbs', None)
            if nxt is not None and absorbs is not None and isinstance(layer, Layer) and absorbs(nxt, x):
                # the two layers as one call: nothing else can read what passes between them here
                x = layer(x, training=training, then=nxt)
                k += 2
                continue
            x = layer(x) if not isinstance(layer, Layer) else layer(x, training=training)
            k += 1
        return x
