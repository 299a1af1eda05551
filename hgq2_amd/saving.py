"""Saving and loading: the variable layout and the layer configurations of the reference, in a container this
environment can write.

The reference saves through Keras (``model.save('*.keras')``, ``save_weights('*.weights.h5')``; its first layer test is
save -> load -> equal outputs, reference tests/base.py:184-201).  What has to survive is

* every variable under the name and dtype the reference gives it: a layer's ``kernel`` / ``bias`` (and ``bn_gamma``,
  ``moving_mean``, ``moving_variance``), ``beta`` (float32 scalar) and ``ebops`` (uint32 scalar)
  (reference src/hgq/layers/core/base.py:188-206); a fixed-point quantizer's ``k`` (uint8), ``i``, ``f`` or ``b`` and, for
  WRAP quantizers, ``i_decay_speed`` (reference src/hgq/quantizer/internal/fixed_point_quantizer.py:215-242,371-399 and
  :48-55 of the same file);
* every layer's ``get_config()`` (constructor keywords, quantizer configurations with their constraints and regularizers).

A variable's key is its Keras-style path: the names of the layers it is nested in, then the variable name, joined by
``/`` (``q_dense/q_dense_iq/fixed_point_quantizer_kif/f``).  The container is a NumPy ``.npz`` (one array per variable,
dtypes kept, no pickling on load) plus, for whole models, the JSON configuration under ``__config__``.  HDF5 files
(``.h5`` / ``.keras``) need ``h5py``, which is not installed here; the mapping below is what such a reader / writer
would iterate over.
"""

from __future__ import annotations

import json

import numpy as np
import torch
from torch import nn

from . import constraints as _constraints
from . import core as _core
from . import regularizers as _regularizers
from .quantizer.config import QuantizerConfig

_NP_DTYPES = {torch.float32: np.float32, torch.uint8: np.uint8, torch.uint32: np.uint32, torch.int32: np.int32}


# --------------------------------------------------------------------------------------------------------------
# variables
# --------------------------------------------------------------------------------------------------------------
def variable_paths(model) -> dict[str, torch.Tensor]:
    """``{path: variable}`` for every variable of ``model`` (built layers only), in creation order per layer."""
    parents: dict[int, nn.Module | None] = {id(model): None}
    for m in model.modules():
        for child in m.children():
            parents.setdefault(id(child), m)  # a shared sub-layer keeps the first parent that holds it
    out: dict[str, torch.Tensor] = {}
    for m in model.modules():
        if not isinstance(m, _core.Layer):
            continue
        chain, cur = [], m
        while cur is not None:
            if isinstance(cur, _core.Layer):
                chain.append(cur.name)
            cur = parents.get(id(cur))
        prefix = '/'.join(reversed(chain))
        own = list(m._parameters.items()) + list(m._buffers.items())
        for attr, t in own:
            if t is None or not attr.startswith('_var_'):
                continue
            path = f'{prefix}/{attr[len("_var_"):]}'
            if path in out:
                raise ValueError(f'two variables share the path {path}: give the layers distinct names')
            out[path] = t
    return out


def _to_numpy(t: torch.Tensor) -> np.ndarray:
    t = t.detach().cpu()
    if t.dtype == torch.uint32:  # numpy conversion of uint32 tensors goes through the bit pattern
        return t.view(torch.int32).numpy().view(np.uint32).copy()
    return t.numpy().copy()


def _assign(t: torch.Tensor, a: np.ndarray, path: str):
    want = _NP_DTYPES.get(t.dtype)
    if want is None or a.dtype != want:
        raise ValueError(f'{path}: stored dtype {a.dtype}, the variable is {t.dtype}')
    if tuple(a.shape) != tuple(t.shape):
        raise ValueError(f'{path}: stored shape {tuple(a.shape)}, the variable is {tuple(t.shape)}')
    src = torch.from_numpy(a.view(np.int32) if a.dtype == np.uint32 else a)
    with torch.no_grad():
        (t.view(torch.int32) if t.dtype == torch.uint32 else t).copy_(src.to(t.device))


def save_weights(model, file):
    """Every variable of a built model into an ``.npz`` keyed by variable path."""
    arrays = {path: _to_numpy(t) for path, t in variable_paths(model).items()}
    np.savez(file, **arrays)


def load_weights(model, file, strict: bool = True):
    """Assign the variables of a built model from an ``.npz`` written by :func:`save_weights` (or by any writer that uses
    the same paths and dtypes).  ``strict``: every variable must be present and nothing else."""
    with np.load(file, allow_pickle=False) as data:
        stored = {k: data[k] for k in data.files if not k.startswith('__')}
    _assign_all(model, stored, strict)


def _assign_all(model, stored: dict, strict: bool):
    from . import ops

    variables = variable_paths(model)
    missing = [p for p in variables if p not in stored]
    extra = [p for p in stored if p not in variables]
    if strict and (missing or extra):
        raise KeyError(f'variables missing from the file: {missing}; entries without a variable: {extra}')
    for path, t in variables.items():
        if path in stored:
            _assign(t, stored[path], path)
    ops.touch_state()


# --------------------------------------------------------------------------------------------------------------
# configurations
# --------------------------------------------------------------------------------------------------------------
def _registry():
    from . import host, layers
    from .quantizer import Quantizer

    reg = {name: getattr(layers, name) for name in layers.__all__ if isinstance(getattr(layers, name), type)}
    reg.update({'Sequential': _core.Sequential, 'Quantizer': Quantizer, 'MaxPooling2D': host.MaxPooling2D,
                'AveragePooling2D': host.AveragePooling2D, 'Flatten': host.Flatten, 'GlobalAveragePooling1D': host.GlobalAveragePooling1D})
    return reg


_VALUE_CLASSES = {
    'MinMax': _constraints.MinMax, 'Min': _constraints.Min, 'Max': _constraints.Max, 'ConstantConstraint': _constraints.Constant,
    'MonoL1': _regularizers.MonoL1, 'Constant': _core.Constant, 'GlorotUniform': _core.GlorotUniform,
}


def serialize(obj):
    """Configuration value -> JSON-able structure (nested ``{'class_name', 'config'}`` records, like Keras')."""
    if obj is None or isinstance(obj, (bool, int, str)):
        return obj
    if isinstance(obj, float):
        return obj if np.isfinite(obj) else {'class_name': '__float__', 'config': repr(obj)}
    if isinstance(obj, (np.integer, np.floating)):
        return serialize(obj.item())
    if isinstance(obj, (tuple, list)):
        return {'class_name': '__tuple__' if isinstance(obj, tuple) else '__list__', 'config': [serialize(v) for v in obj]}
    if isinstance(obj, dict):
        return {'class_name': '__dict__', 'config': {k: serialize(v) for k, v in obj.items()}}
    if isinstance(obj, QuantizerConfig):
        return {'class_name': 'QuantizerConfig', 'config': {k: serialize(v) for k, v in obj.get_config().items()}}
    if isinstance(obj, _constraints.Constant):
        return {'class_name': 'ConstantConstraint', 'config': serialize(obj.get_config())['config']}
    for name, cls in _VALUE_CLASSES.items():
        if type(obj) is cls:
            cfg = obj.get_config() if hasattr(obj, 'get_config') else dict(vars(obj))
            return {'class_name': name, 'config': {k: serialize(v) for k, v in cfg.items()}}
    if isinstance(obj, _core.Layer):
        return {'class_name': type(obj).__name__, 'config': {k: serialize(v) for k, v in obj.get_config().items()}}
    raise TypeError(f'cannot serialize {type(obj).__name__}: {obj!r}')


def deserialize(rec):
    if not isinstance(rec, dict):
        return rec
    name, cfg = rec['class_name'], rec['config']
    if name == '__float__':
        return float(cfg)
    if name == '__tuple__':
        return tuple(deserialize(v) for v in cfg)
    if name == '__list__':
        return [deserialize(v) for v in cfg]
    if name == '__dict__':
        return {k: deserialize(v) for k, v in cfg.items()}
    kwargs = {k: deserialize(v) for k, v in cfg.items()}
    if name == 'QuantizerConfig':
        return QuantizerConfig(**kwargs)
    if name in _VALUE_CLASSES:
        return _VALUE_CLASSES[name](**kwargs)
    reg = _registry()
    if name in reg:
        return reg[name].from_config(kwargs)
    raise ValueError(f'unknown class {name!r} in a saved configuration')


def save_model(model, file, input_shape=None):
    """Configuration + variables of a built model.  ``input_shape`` (batch axis included, ``None`` allowed there) is what
    :func:`load_model` builds the layers with before it assigns the variables; it defaults to the shape the model was last
    called with."""
    shape = input_shape if input_shape is not None else getattr(model, '_last_input_shape', None)
    if shape is None:
        raise ValueError('input_shape is needed: the model has not been called yet')
    arrays = {path: _to_numpy(t) for path, t in variable_paths(model).items()}
    arrays['__config__'] = np.array(json.dumps(serialize(model)))
    arrays['__input_shape__'] = np.array(json.dumps([None if s is None else int(s) for s in shape]))
    np.savez(file, **arrays)


def load_model(file, device=None):
    """Rebuild a model saved by :func:`save_model`: same classes and configurations, variables assigned bit for bit."""
    with np.load(file, allow_pickle=False) as data:
        config = json.loads(str(data['__config__']))
        shape = tuple(json.loads(str(data['__input_shape__'])))
        stored = {k: data[k] for k in data.files if not k.startswith('__')}
    prev = _core._default_device
    if device is not None:
        _core.set_default_device(device)
    try:
        model = deserialize(config)
        build_for_shape(model, shape)
    finally:
        _core.set_default_device(prev)
    _assign_all(model, stored, True)
    model._last_input_shape = shape
    return model


def build_for_shape(model, input_shape):
    """Create the variables of ``model`` for ``input_shape`` without running a forward pass."""
    shape = tuple(input_shape)
    if isinstance(model, _core.Sequential):
        for layer in model.layers:
            if isinstance(layer, _core.Layer):
                if not layer.built:
                    layer.build(shape)
                    layer.built = True
                shape = tuple(layer.compute_output_shape(shape))
        model.built = True
        return shape
    if not model.built:
        model.build(shape)
        model.built = True
    return tuple(model.compute_output_shape(shape))
