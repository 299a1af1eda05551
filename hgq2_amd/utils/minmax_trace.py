"""Calibration pass for WRAP quantizers (reference src/hgq/utils/minmax_trace.py:13-99): run a
dataset through the model with ``training='tracing'`` so that every WRAP quantizer widens its
integer bits to what the data needs and records whether it saw negative values."""

from __future__ import annotations

from collections.abc import Sequence

import numpy as np
import torch

from ..core import Layer, TrainingFlagWrapper


def _reset_minmax(layer):
    """``_i <- -1e9`` and ``_k <- 0`` on every trainable WRAP quantizer below ``layer`` (reference :13-21)."""
    for m in layer.modules():
        if hasattr(m, '_i_decay_speed') and getattr(m, 'trainable', True):
            with torch.no_grad():
                m._i.fill_(-1e9)
                m._k.zero_()


def _batches(data, batch_size):
    """Mirror of the reference's ``Dataset(data, batch_size, shuffle=False)``: yields the model inputs."""
    if isinstance(data, (tuple, list)) and not torch.is_tensor(data):
        n = len(data[0])
        for s in range(0, n, batch_size):
            yield tuple(d[s:s + batch_size] for d in data)
    else:
        n = len(data)
        for s in range(0, n, batch_size):
            yield data[s:s + batch_size]


def _to_device(x, device):
    if isinstance(x, tuple):
        return tuple(_to_device(t, device) for t in x)
    return torch.as_tensor(np.asarray(x) if not torch.is_tensor(x) else x, dtype=torch.float32).to(device)


def trace_minmax(model: Layer, data, reset: bool = True, batch_size: int = 1024, verbose: int | bool = 0,
                 return_results: bool = False, device=None):
    """With a calibration dataset, find the integer bits the WRAP quantizers of ``model`` need.

    Parameters follow the reference: ``data`` is an array (or a sequence of arrays for multi-input
    models), ``reset`` clears the traced state first, ``verbose`` prints the per-layer EBOPs,
    ``return_results`` returns the model outputs on the data instead of the total EBOPs.
    ``device`` (extra): where the batches are placed; defaults to the model's device.
    """
    if device is None:
        p = next(iter(model.parameters()), None)
        device = p.device if p is not None else torch.device('cuda', torch.cuda.current_device())
    if reset:
        _reset_minmax(model)
    results = []
    flag = TrainingFlagWrapper('tracing')
    with torch.no_grad():
        for batch in _batches(data, batch_size):
            x = _to_device(batch, device)
            r = model(*x, training=flag) if isinstance(x, tuple) else model(x, training=flag)
            if return_results:
                results.append(tuple(t.cpu().numpy() for t in r) if isinstance(r, (tuple, list)) else r.cpu().numpy())
    record: dict[str, int] = {}
    layers = getattr(model, 'layers', None)
    for layer in (layers if layers is not None else [model]):
        if getattr(layer, 'enable_ebops', False):
            e = layer.ebops
            record[layer.name] = int(e.cpu().view(torch.int32)) if torch.is_tensor(e) else int(e)
    if verbose and record:
        width = max(max(map(len, record.keys())), 5)
        for k, v in record.items():
            print(f'{k:{width}}: {v}')
        print(f'Total: {sum(record.values())}')
    if return_results:
        if results and isinstance(results[0], tuple):
            return tuple(np.concatenate([r[i] for r in results]) for i in range(len(results[0])))
        return np.concatenate(results)
    return int(sum(record.values()))
